// Forge loop for the matvec operators: candidate schedules -> run -> gate against
// an FP64 oracle -> time -> measured selection -> cache.
//
// Mirrors the reference's per-candidate loop (rust/crates/lev-cli/src/main.rs:
// 1941-2024, `vk_q4k`): x = SplitMix64(0x4C455649).next_signed_unit(), every
// candidate is gated with max|y - oracle| / max(1, |oracle|) < 1e-4
// (lev-cpu/src/lib.rs:341-353), timed with 3 warm and 11 timed samples, and a
// candidate other than the baseline (candidate 0) is selected only if its median
// beats the baseline's by more than 2 %.  The reference compiles an emitted
// shader per candidate and caches the binary by source hash; here a candidate is
// a precompiled kernel variant of the library (lev_hip_forge_candidates) and the
// cache holds the selection, keyed by operator, shape, device name, ABI version and
// a hash of this build's candidate table for the shape; a cached selection is gated
// again (one launch) before it is installed.  Candidates are timed over rotating
// copies of the weights, so that a matrix that fits the last-level cache is timed as
// decode meets it: from HBM.  The FP64 products below follow matvec_q4k_f64 / dequant_block_f64
// (lev-cpu/src/lib.rs:134-195) and Q4Oracle.matvecFP64 (Q4Lowering.swift:1215);
// they only accept or reject a candidate and never supply an output.
#pragma once

#include <algorithm>
#include <chrono>
#include <cmath>
#include <fstream>
#include <sstream>

#include "leviathan_hip.hpp"

namespace leviathan {

struct ForgeCandidate {
    lev_schedule schedule{};
    double medianUs = 0;
    double maxRelErr = 0;   // negative: rejected (count mismatch or a non-finite value)
    bool pass = false;
};

struct ForgeReport {
    uint32_t op = 0;
    int64_t inDim = 0, rows = 0, ncol = 1;
    std::string device;
    std::vector<ForgeCandidate> candidates;   // candidate 0 is the baseline
    int selected = -1;                        // index into candidates; -1: the baseline failed the gate
    bool fromCache = false;
    std::string describe() const {
        std::ostringstream o;
        for (size_t i = 0; i < candidates.size(); ++i) {
            const ForgeCandidate &c = candidates[i];
            o << (int(i) == selected ? "* " : "  ") << "family=" << c.schedule.family
              << " rows_in_flight=" << c.schedule.rows_in_flight << " persistent=" << c.schedule.persistent
              << " max_rel_err=" << c.maxRelErr << " median_us=" << c.medianUs << (c.pass ? " PASS" : " FAIL")
              << "\n";
        }
        return o.str();
    }
};

struct ForgeOptions {
    int warm = 3, timed = 11;     // samples, as run_q4k_matvec(…, 3, 11)
    int launchesPerSample = 20;   // launches per sample (a single GEMV launch is a few microseconds)
    double gate = 1e-4;
    double margin = 0.02;         // a non-baseline candidate must be more than this much faster
    uint64_t seed = 0x4C455649ull;
    std::string cachePath;        // empty: no cache
    size_t rotateBytes = (size_t)512 << 20;   // weight copies cycled through while timing (at most 64)
    // Q4_K and Q6_K: forge the int8-activation GEMV (lev_hip_q4_k_gemv_q8,
    // lev_hip_q6_k_gemv_q8) instead of the f32 one.  The activations are quantised on the device and the oracle is the FP64
    // product over those same codes (q * d), as `lev vk-q8` gates it
    // (lev-cli/src/main.rs:1788-1868).
    bool int8Activations = false;
};

namespace forge_detail {

struct SplitMix64 {   // lev-cpu/src/lib.rs:355-372
    uint64_t s;
    uint64_t next() {
        s += 0x9E3779B97F4A7C15ull;
        uint64_t z = s;
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        return z ^ (z >> 31);
    }
    float nextSignedUnit() {
        float u = (float)(next() >> 40) / (float)(1ull << 24);
        return u * 2.0f - 1.0f;
    }
};

inline double halfToDouble(uint16_t h) {
    const int sign = h >> 15, exp = (h >> 10) & 31, man = h & 1023;
    double v;
    if (exp == 0) v = std::ldexp((double)man, -24);
    else if (exp == 31) v = man ? NAN : INFINITY;
    else v = std::ldexp((double)(man | 1024), exp - 25);
    return sign ? -v : v;
}

inline void q4_0RowF64(const uint8_t *row, int64_t inDim, const float *x, double &sum) {
    for (int64_t b = 0; b < inDim / 32; ++b) {
        const uint8_t *blk = row + b * 18;
        const double d = halfToDouble((uint16_t)(blk[0] | blk[1] << 8));
        for (int l = 0; l < 16; ++l) {
            sum += d * ((double)(blk[2 + l] & 0xF) - 8.0) * (double)x[b * 32 + l];
            sum += d * ((double)(blk[2 + l] >> 4) - 8.0) * (double)x[b * 32 + 16 + l];
        }
    }
}

inline void q4_kRowF64(const uint8_t *row, int64_t inDim, const float *x, double &sum) {
    for (int64_t b = 0; b < inDim / 256; ++b) {
        const uint8_t *blk = row + b * 144, *s = blk + 4, *qs = blk + 16;
        const double d = halfToDouble((uint16_t)(blk[0] | blk[1] << 8));
        const double dmin = halfToDouble((uint16_t)(blk[2] | blk[3] << 8));
        for (int j = 0; j < 8; ++j) {
            int sc, mn;   // unpack_scale_min, lev-cpu/src/lib.rs:64-74
            if (j < 4) {
                sc = s[j] & 63;
                mn = s[j + 4] & 63;
            } else {
                sc = (s[j + 4] & 0xF) | ((s[j - 4] >> 6) << 4);
                mn = (s[j + 4] >> 4) | ((s[j] >> 6) << 4);
            }
            const double d1 = d * sc, mm = dmin * mn;
            const uint8_t *q = qs + (j / 2) * 32;
            for (int l = 0; l < 32; ++l) {
                const int code = (j & 1) ? q[l] >> 4 : q[l] & 0xF;
                sum += (d1 * code - mm) * (double)x[b * 256 + j * 32 + l];
            }
        }
    }
}

// q6k_unpack + matvec_q6k_f64, lev-cpu/src/lib.rs:203-300
inline void q6_kRowF64(const uint8_t *row, int64_t inDim, const float *x, double &sum) {
    for (int64_t b = 0; b < inDim / 256; ++b) {
        const uint8_t *blk = row + b * 210, *ql = blk, *qh = blk + 128;
        const int8_t *sc = reinterpret_cast<const int8_t *>(blk + 192);
        const double d = halfToDouble((uint16_t)(blk[208] | blk[209] << 8));
        for (int half = 0; half < 2; ++half)
            for (int l = 0; l < 32; ++l) {
                const int is = l / 16, h = qh[32 * half + l];
                const int q1 = ((ql[64 * half + l] & 0xF) | ((h & 3) << 4)) - 32;
                const int q2 = ((ql[64 * half + 32 + l] & 0xF) | (((h >> 2) & 3) << 4)) - 32;
                const int q3 = ((ql[64 * half + l] >> 4) | (((h >> 4) & 3) << 4)) - 32;
                const int q4 = ((ql[64 * half + 32 + l] >> 4) | (((h >> 6) & 3) << 4)) - 32;
                const float *xb = x + b * 256 + 128 * half;
                const int8_t *s8 = sc + 8 * half;
                sum += d * s8[is] * q1 * (double)xb[l];
                sum += d * s8[is + 2] * q2 * (double)xb[32 + l];
                sum += d * s8[is + 4] * q3 * (double)xb[64 + l];
                sum += d * s8[is + 6] * q4 * (double)xb[96 + l];
            }
    }
}
inline double maxRelErr(const std::vector<float> &got, const std::vector<double> &ref) {
    if (got.size() != ref.size() || got.empty()) return -1.0;
    double worst = 0;
    for (size_t i = 0; i < got.size(); ++i) {
        if (!std::isfinite(got[i]) || !std::isfinite(ref[i])) return -1.0;
        worst = std::max(worst, std::fabs((double)got[i] - ref[i]) / std::max(1.0, std::fabs(ref[i])));
    }
    return worst;
}

// FNV-1a over the candidate table: a build whose variants differ has different keys
inline uint64_t tableHash(const lev_schedule *list, uint32_t n) {
    uint64_t h = 0xcbf29ce484222325ull;
    auto mix = [&](uint32_t v) {
        for (int i = 0; i < 4; ++i) {
            h ^= (v >> (8 * i)) & 0xFFu;
            h *= 0x100000001b3ull;
        }
    };
    mix(n);
    for (uint32_t i = 0; i < n; ++i) {
        mix(list[i].op);
        mix(list[i].family);
        mix(list[i].rows_in_flight);
        mix(list[i].persistent);
    }
    return h;
}
inline std::string cacheKey(uint32_t op, int64_t inDim, int64_t rows, int64_t ncol, std::string device,
                            uint64_t table) {
    std::replace(device.begin(), device.end(), ' ', '_');
    std::ostringstream k;
    k << "leviathan-forge-2 " << lev_hip_abi_version() << " " << device << " " << table << " " << op << " "
      << inDim << " " << rows << " " << ncol;
    return k.str();
}
inline double median(std::vector<double> v) {
    if (v.empty()) return 0;
    std::sort(v.begin(), v.end());
    return v[v.size() / 2];
}
// candidate 0 must pass; the fastest passing candidate wins if it beats it by more than the margin
inline int choose(const std::vector<ForgeCandidate> &c, double margin) {
    if (c.empty() || !c[0].pass) return -1;
    size_t best = 0;
    for (size_t i = 1; i < c.size(); ++i)
        if (c[i].pass && c[i].medianUs < c[best].medianUs) best = i;
    return best != 0 && c[best].medianUs < c[0].medianUs * (1.0 - margin) ? (int)best : 0;
}

}  // namespace forge_detail

class MatvecForge {
public:
    // `weights`: rows x inDim in the tensor's GGUF block layout (Q4_0, Q4_K or Q6_K),
    // as read from the file.  Leaves the selection installed on the runner's
    // context (or the built-in choice, when that won) and returns the report.
    static ForgeReport forge(Runner &r, GGMLTensorType type, const std::vector<uint8_t> &weights, int64_t rows,
                             int64_t inDim, int64_t ncol = 1, const ForgeOptions &opt = ForgeOptions()) {
        using namespace forge_detail;
        if (type != GGMLTensorType::q4_0 && type != GGMLTensorType::q4_K && type != GGMLTensorType::q6_K)
            throw Gemma4Error(Gemma4Error::badTensorGeometry, "forge: Q4_0, Q4_K and Q6_K matvecs have schedules");
        if (opt.int8Activations && type == GGMLTensorType::q4_0)
            throw Gemma4Error(Gemma4Error::badTensorGeometry, "forge: the int8-activation GEMVs are Q4_K and Q6_K");
        const bool q6 = type == GGMLTensorType::q6_K;
        const uint32_t op = type == GGMLTensorType::q4_0 ? LEV_OP_Q4_0_GEMV
                            : q6 ? (opt.int8Activations ? LEV_OP_Q6_K_GEMV_Q8 : LEV_OP_Q6_K_GEMV)
                                 : (opt.int8Activations ? LEV_OP_Q4_K_GEMV_Q8 : LEV_OP_Q4_K_GEMV);
        const int64_t per = elementsPerBlock(type), bpb = bytesPerBlock(type);
        if (rows <= 0 || inDim <= 0 || ncol <= 0 || inDim % per != 0 ||
            (int64_t)weights.size() != rows * (inDim / per) * bpb)
            throw Gemma4Error(Gemma4Error::badTensorGeometry, "forge: weight bytes do not match rows x inDim");
        lev_ctx *ctx = r.context();
        ForgeReport rep;
        rep.op = op;
        rep.inDim = inDim;
        rep.rows = rows;
        rep.ncol = ncol;
        char name[256] = {0};
        check(ctx, lev_hip_device_name(ctx, name, sizeof name));
        rep.device = name;
        lev_schedule list[16];
        uint32_t n = 0;
        check(ctx, lev_hip_forge_candidates(ctx, op, (uint32_t)inDim, (uint32_t)rows, (uint32_t)ncol, list, 16, &n));
        n = std::min<uint32_t>(n, 16);
        const std::string key = cacheKey(op, inDim, rows, ncol, rep.device, tableHash(list, n));

        // inputs, oracle and the launch closure (also needed to gate a cached selection)
        SplitMix64 rng{opt.seed};
        std::vector<float> x((size_t)(inDim * ncol));
        for (float &v : x) v = rng.nextSignedUnit();
        std::vector<double> ref((size_t)(rows * ncol), 0.0);
        const int64_t rowBytes = inDim / per * bpb;
        size_t copies = weights.empty() ? 1 : opt.rotateBytes / weights.size();
        copies = std::max<size_t>(1, std::min<size_t>(copies, 64));
        std::vector<DeviceBuffer> dws;
        for (size_t k = 0; k < copies; ++k) dws.push_back(r.makeBuffer(weights));
        DeviceBuffer dx = r.makeBuffer(x), dy = r.makeBuffer(rows * ncol * 4);
        DeviceBuffer dxq, dxs;
        if (opt.int8Activations) {
            // quantise on the device, then continue with the values the codes stand for
            dxq = r.makeBuffer(inDim * ncol);
            dxs = r.makeBuffer(inDim / 32 * ncol * 8);
            check(ctx, lev_hip_norm_quant_q8(ctx, dx.floats(), x.size(), nullptr, nullptr, 0.f,
                                             static_cast<int8_t *>(dxq.contents()), dxs.floats(), nullptr,
                                             (uint32_t)inDim, (uint32_t)ncol));
            check(ctx, lev_hip_sync(ctx));
            const std::vector<int8_t> q = r.read<int8_t>(dxq, (size_t)(inDim * ncol));
            const std::vector<float> ds = r.read<float>(dxs, (size_t)(inDim / 32 * ncol * 2));
            for (size_t i = 0; i < x.size(); ++i) x[i] = (float)q[i] * ds[(i / 32) * 2];
        }
        for (int64_t c = 0; c < ncol; ++c)
            for (int64_t i = 0; i < rows; ++i) {
                double s = 0;
                const uint8_t *row = weights.data() + i * rowBytes;
                if (op == LEV_OP_Q4_0_GEMV) q4_0RowF64(row, inDim, x.data() + c * inDim, s);
                else if (q6) q6_kRowF64(row, inDim, x.data() + c * inDim, s);
                else q4_kRowF64(row, inDim, x.data() + c * inDim, s);
                ref[(size_t)(c * rows + i)] = s;
            }
        size_t turn = 0;
        auto launch = [&]() {
            const DeviceBuffer &dw = dws[turn++ % copies];
            const size_t yn = (size_t)(rows * ncol);
            switch (op) {
            case LEV_OP_Q4_K_GEMV_Q8:
                return lev_hip_q4_k_gemv_q8(ctx, dw.contents(), weights.size(), 0,
                                            static_cast<const int8_t *>(dxq.contents()), dxs.floats(), x.size(),
                                            dy.floats(), yn, (uint32_t)inDim, (uint32_t)rows, (uint32_t)ncol);
            case LEV_OP_Q6_K_GEMV_Q8:
                return lev_hip_q6_k_gemv_q8(ctx, dw.contents(), weights.size(), 0,
                                            static_cast<const int8_t *>(dxq.contents()), dxs.floats(), x.size(),
                                            dy.floats(), yn, (uint32_t)inDim, (uint32_t)rows, (uint32_t)ncol);
            case LEV_OP_Q4_0_GEMV:
                return lev_hip_q4_0_gemv(ctx, dw.contents(), weights.size(), 0, dx.floats(), (size_t)inDim,
                                         dy.floats(), (size_t)rows, (uint32_t)inDim, (uint32_t)rows);
            case LEV_OP_Q6_K_GEMV:
                return lev_hip_q6_k_gemv(ctx, dw.contents(), weights.size(), 0, dx.floats(), (size_t)inDim,
                                         dy.floats(), (size_t)rows, (uint32_t)inDim, (uint32_t)rows, nullptr, nullptr);
            default:
                return lev_hip_q4_k_gemv_ncol(ctx, dw.contents(), weights.size(), 0, dx.floats(), x.size(), nullptr,
                                              0.f, dy.floats(), yn, (uint32_t)inDim, (uint32_t)rows, (uint32_t)ncol);
            }
        };
        // one launch into a poisoned output (a candidate that writes nothing cannot pass on
        // the previous one's result), compared with the oracle
        auto gate = [&](const lev_schedule &sch) {
            check(ctx, lev_hip_forge_select(ctx, (uint32_t)inDim, (uint32_t)rows, (uint32_t)ncol, &sch));
            std::vector<float> poison((size_t)(rows * ncol), NAN);
            check(ctx, lev_hip_buf_upload(ctx, dy.contents(), poison.data(), poison.size() * 4));
            check(ctx, launch());
            check(ctx, lev_hip_sync(ctx));
            return maxRelErr(r.read<float>(dy, (size_t)(rows * ncol)), ref);
        };

        if (!opt.cachePath.empty()) {
            std::ifstream in(opt.cachePath);
            std::string line;
            while (std::getline(in, line)) {
                if (line.compare(0, key.size() + 1, key + " ") != 0) continue;
                std::istringstream f(line.substr(key.size() + 1));
                ForgeCandidate c;
                c.schedule.op = op;
                int baseline = 0;
                if (!(f >> c.schedule.family >> c.schedule.rows_in_flight >> c.schedule.persistent >> c.medianUs >>
                      c.maxRelErr >> baseline))
                    continue;
                bool legal = false;
                for (uint32_t i = 0; i < n; ++i)
                    legal = legal || (list[i].family == c.schedule.family &&
                                      list[i].rows_in_flight == c.schedule.rows_in_flight &&
                                      list[i].persistent == c.schedule.persistent);
                if (!legal) continue;
                // the cached choice is gated again by this build before it is installed
                c.maxRelErr = gate(c.schedule);
                c.pass = c.maxRelErr >= 0 && c.maxRelErr < opt.gate;
                if (!c.pass) continue;
                rep.candidates.push_back(c);
                rep.selected = 0;
                rep.fromCache = true;
                install(ctx, rep, baseline != 0);
                return rep;
            }
        }
        for (uint32_t i = 0; i < n; ++i) {
            ForgeCandidate c;
            c.schedule = list[i];
            c.maxRelErr = gate(list[i]);
            c.pass = c.maxRelErr >= 0 && c.maxRelErr < opt.gate;
            std::vector<double> samples;
            for (int s = 0; s < opt.warm + opt.timed; ++s) {
                auto t0 = std::chrono::steady_clock::now();
                for (int k = 0; k < opt.launchesPerSample; ++k) check(ctx, launch());
                check(ctx, lev_hip_sync(ctx));
                auto t1 = std::chrono::steady_clock::now();
                if (s >= opt.warm)
                    samples.push_back(std::chrono::duration<double, std::micro>(t1 - t0).count() /
                                      opt.launchesPerSample);
            }
            c.medianUs = median(samples);
            rep.candidates.push_back(c);
        }
        rep.selected = choose(rep.candidates, opt.margin);
        install(ctx, rep, rep.selected <= 0);
        if (!opt.cachePath.empty() && rep.selected >= 0) {
            const ForgeCandidate &c = rep.candidates[(size_t)rep.selected];
            std::ofstream out(opt.cachePath, std::ios::app);
            out << key << " " << c.schedule.family << " " << c.schedule.rows_in_flight << " " << c.schedule.persistent
                << " " << c.medianUs << " " << c.maxRelErr << " " << (rep.selected == 0 ? 1 : 0) << "\n";
        }
        return rep;
    }

private:
    friend class MoELayerForge;
    static void check(lev_ctx *ctx, int st) {
        if (st != LEV_OK)
            throw Gemma4Error(Gemma4Error::commandFailed, std::string("forge: ") + lev_hip_last_error(ctx));
    }
    // the baseline is the built-in choice: nothing stays installed for it
    static void install(lev_ctx *ctx, const ForgeReport &rep, bool baseline) {
        if (baseline || rep.selected < 0)
            check(ctx, lev_hip_forge_clear(ctx, rep.op, (uint32_t)rep.inDim, (uint32_t)rep.rows, (uint32_t)rep.ncol));
        else
            check(ctx, lev_hip_forge_select(ctx, (uint32_t)rep.inDim, (uint32_t)rep.rows, (uint32_t)rep.ncol,
                                            &rep.candidates[(size_t)rep.selected].schedule));
    }
};

// The MoE layer at one to four tokens (MoELoweringForge.forge, MoELowering.swift:1896-1985:
// derive the lowered layer's candidates, gate each against the FP64 oracle, time, select).
// The gate has two parts, as the layer has two contracts: the routing must be a top-k of
// the FP64 router probabilities (ties within 1e-6 may fall either way), and the output must
// agree with the FP64 expert chain evaluated on the routing the device chose.
class MoELayerForge {
public:
    // `pool`: the bytes `binding`'s offsets refer to; `router`: F32 [experts][hidden].
    static ForgeReport forge(Runner &r, const std::vector<uint8_t> &pool, const MoEBinding &binding,
                             const std::vector<float> &router, int tokens, const ForgeOptions &opt = ForgeOptions()) {
        using namespace forge_detail;
        const int H = binding.hidden, I = binding.expertIntermediate, E = binding.experts, K = binding.topK;
        if (H <= 0 || I <= 0 || E <= 0 || K <= 0 || K > E || H % 32 || I % 32 || tokens < 1 || tokens > 4 ||
            (int64_t)router.size() != (int64_t)E * H)
            throw Gemma4Error(Gemma4Error::badTensorGeometry, "forge: MoE layer dims");
        lev_ctx *ctx = r.context();
        ForgeReport rep;
        rep.op = LEV_OP_MOE_LAYER_Q4_0;
        rep.inDim = H;
        rep.rows = I;
        rep.ncol = tokens;
        char name[256] = {0};
        MatvecForge::check(ctx, lev_hip_device_name(ctx, name, sizeof name));
        rep.device = name;
        lev_schedule list[16];
        uint32_t n = 0;
        MatvecForge::check(ctx, lev_hip_forge_candidates(ctx, rep.op, (uint32_t)H, (uint32_t)I, (uint32_t)tokens, list,
                                                         16, &n));
        n = std::min<uint32_t>(n, 16);

        SplitMix64 rng{opt.seed};
        std::vector<float> x((size_t)tokens * H);
        for (float &v : x) v = rng.nextSignedUnit();
        // FP64 router probabilities per token
        std::vector<std::vector<double>> prob((size_t)tokens, std::vector<double>((size_t)E));
        for (int t = 0; t < tokens; ++t) {
            double top = -INFINITY, den = 0;
            for (int e = 0; e < E; ++e) {
                double s = 0;
                for (int i = 0; i < H; ++i) s += (double)router[(size_t)e * H + i] * (double)x[(size_t)t * H + i];
                prob[(size_t)t][(size_t)e] = s;
                top = std::max(top, s);
            }
            for (double &p : prob[(size_t)t]) den += (p = std::exp(p - top));
            for (double &p : prob[(size_t)t]) p /= den;
        }
        size_t copies = pool.empty() ? 1 : opt.rotateBytes / pool.size();
        copies = std::max<size_t>(1, std::min<size_t>(copies, 8));
        std::vector<DeviceBuffer> pools;
        for (size_t k = 0; k < copies; ++k) pools.push_back(r.makeBuffer(pool));
        DeviceBuffer dr = r.makeBuffer(router), dx = r.makeBuffer(x), dy = r.makeBuffer((int64_t)tokens * H * 4),
                     dids = r.makeBuffer((int64_t)tokens * K * 4), dwts = r.makeBuffer((int64_t)tokens * K * 4);
        size_t turn = 0;
        auto launch = [&]() {
            lev_moe_experts p;
            p.d_base = pools[turn++ % copies].contents();
            p.base_bytes = pool.size();
            p.gate_off = (uint64_t)binding.gateOffset;
            p.up_off = (uint64_t)binding.upOffset;
            p.down_off = (uint64_t)binding.downOffset;
            p.gate_stride = (uint64_t)binding.gateStride;
            p.up_stride = (uint64_t)binding.upStride;
            p.down_stride = (uint64_t)binding.downStride;
            p.hidden = (uint32_t)H;
            p.inter = (uint32_t)I;
            p.experts = (uint32_t)E;
            return lev_hip_moe_layer_q4_0(ctx, &p, dr.floats(), nullptr, dx.floats(), dy.floats(),
                                          static_cast<int32_t *>(dids.contents()), dwts.floats(), (uint32_t)K,
                                          (uint32_t)tokens);
        };
        // FP64 expert chain on a given routing (runMoeBatchedRouted, Gemma4.swift:2073; g4_gelu_up :4364-4388)
        auto chain = [&](int t, const int32_t *ids, const float *wts, std::vector<double> &y) {
            y.assign((size_t)H, 0.0);
            const int64_t guRow = H / 32 * 18, dnRow = I / 32 * 18;
            std::vector<float> act((size_t)I);
            for (int k = 0; k < K; ++k) {
                const uint8_t *g = pool.data() + binding.gateOffset + (int64_t)ids[k] * binding.gateStride;
                const uint8_t *u = pool.data() + binding.upOffset + (int64_t)ids[k] * binding.upStride;
                const uint8_t *d = pool.data() + binding.downOffset + (int64_t)ids[k] * binding.downStride;
                for (int i = 0; i < I; ++i) {
                    double gs = 0, us = 0;
                    q4_0RowF64(g + i * guRow, H, x.data() + (size_t)t * H, gs);
                    q4_0RowF64(u + i * guRow, H, x.data() + (size_t)t * H, us);
                    const double inner = 0.7978845608028654 * (gs + 0.044715 * gs * gs * gs);
                    act[(size_t)i] = (float)(0.5 * gs * (1.0 + std::tanh(inner)) * us);
                }
                for (int i = 0; i < H; ++i) {
                    double s = 0;
                    q4_0RowF64(d + i * dnRow, I, act.data(), s);
                    y[(size_t)i] += (double)wts[k] * s;
                }
            }
        };
        auto gate = [&](const lev_schedule &sch) {
            MatvecForge::check(ctx, lev_hip_forge_select(ctx, (uint32_t)H, (uint32_t)I, (uint32_t)tokens, &sch));
            std::vector<float> poison((size_t)tokens * H, NAN);
            MatvecForge::check(ctx, lev_hip_buf_upload(ctx, dy.contents(), poison.data(), poison.size() * 4));
            MatvecForge::check(ctx, launch());
            MatvecForge::check(ctx, lev_hip_sync(ctx));
            const std::vector<float> y = r.read<float>(dy, (size_t)tokens * H), wts = r.read<float>(dwts, (size_t)tokens * K);
            const std::vector<int32_t> ids = r.read<int32_t>(dids, (size_t)tokens * K);
            double worst = 0;
            for (int t = 0; t < tokens; ++t) {
                // routing: K distinct experts in range, none of them clearly below an expert left out
                std::vector<char> chosen((size_t)E, 0);
                double least = INFINITY, psum = 0;
                for (int k = 0; k < K; ++k) {
                    const int32_t e = ids[(size_t)t * K + k];
                    if (e < 0 || e >= E || chosen[(size_t)e]) return -1.0;
                    chosen[(size_t)e] = 1;
                    least = std::min(least, prob[(size_t)t][(size_t)e]);
                    psum += prob[(size_t)t][(size_t)e];
                }
                for (int e = 0; e < E; ++e)
                    if (!chosen[(size_t)e] && prob[(size_t)t][(size_t)e] > least + 1e-6) return -1.0;
                for (int k = 0; k < K; ++k)   // renormalised probabilities (Gemma4.swift:3795-3810)
                    worst = std::max(worst, std::fabs((double)wts[(size_t)t * K + k] -
                                                      prob[(size_t)t][(size_t)ids[(size_t)t * K + k]] / psum));
                std::vector<double> ref;
                chain(t, ids.data() + (size_t)t * K, wts.data() + (size_t)t * K, ref);
                const double e = maxRelErr(std::vector<float>(y.begin() + (size_t)t * H, y.begin() + (size_t)(t + 1) * H), ref);
                if (e < 0) return -1.0;
                worst = std::max(worst, e);
            }
            return worst;
        };
        for (uint32_t i = 0; i < n; ++i) {
            ForgeCandidate c;
            c.schedule = list[i];
            c.maxRelErr = gate(list[i]);
            c.pass = c.maxRelErr >= 0 && c.maxRelErr < opt.gate;
            std::vector<double> samples;
            for (int s = 0; s < opt.warm + opt.timed; ++s) {
                auto t0 = std::chrono::steady_clock::now();
                for (int k = 0; k < opt.launchesPerSample; ++k) MatvecForge::check(ctx, launch());
                MatvecForge::check(ctx, lev_hip_sync(ctx));
                auto t1 = std::chrono::steady_clock::now();
                if (s >= opt.warm)
                    samples.push_back(std::chrono::duration<double, std::micro>(t1 - t0).count() /
                                      opt.launchesPerSample);
            }
            c.medianUs = median(samples);
            rep.candidates.push_back(c);
        }
        rep.selected = choose(rep.candidates, opt.margin);
        MatvecForge::install(ctx, rep, rep.selected <= 0);
        return rep;
    }
};

}  // namespace leviathan

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
// cache holds the selection, keyed by operator, shape, device name and ABI
// version.  The FP64 products below follow matvec_q4k_f64 / dequant_block_f64
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
    // Q4_K only: forge the int8-activation GEMV (lev_hip_q4_k_gemv_q8) instead of the
    // f32 one.  The activations are quantised on the device and the oracle is the FP64
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

inline double maxRelErr(const std::vector<float> &got, const std::vector<double> &ref) {
    if (got.size() != ref.size() || got.empty()) return -1.0;
    double worst = 0;
    for (size_t i = 0; i < got.size(); ++i) {
        if (!std::isfinite(got[i]) || !std::isfinite(ref[i])) return -1.0;
        worst = std::max(worst, std::fabs((double)got[i] - ref[i]) / std::max(1.0, std::fabs(ref[i])));
    }
    return worst;
}

inline std::string cacheKey(uint32_t op, int64_t inDim, int64_t rows, int64_t ncol, std::string device) {
    std::replace(device.begin(), device.end(), ' ', '_');
    std::ostringstream k;
    k << "leviathan-forge-1 " << lev_hip_abi_version() << " " << device << " " << op << " " << inDim << " "
      << rows << " " << ncol;
    return k.str();
}

}  // namespace forge_detail

class MatvecForge {
public:
    // `weights`: rows x inDim in the tensor's GGUF block layout (Q4_0 or Q4_K),
    // as read from the file.  Leaves the selection installed on the runner's
    // context (or the built-in choice, when that won) and returns the report.
    static ForgeReport forge(Runner &r, GGMLTensorType type, const std::vector<uint8_t> &weights, int64_t rows,
                             int64_t inDim, int64_t ncol = 1, const ForgeOptions &opt = ForgeOptions()) {
        using namespace forge_detail;
        if (type != GGMLTensorType::q4_0 && type != GGMLTensorType::q4_K)
            throw Gemma4Error(Gemma4Error::badTensorGeometry, "forge: only Q4_0 and Q4_K matvecs have schedules");
        if (opt.int8Activations && type != GGMLTensorType::q4_K)
            throw Gemma4Error(Gemma4Error::badTensorGeometry, "forge: the int8-activation GEMV is Q4_K");
        const uint32_t op = type == GGMLTensorType::q4_0 ? LEV_OP_Q4_0_GEMV
                            : opt.int8Activations       ? LEV_OP_Q4_K_GEMV_Q8
                                                        : LEV_OP_Q4_K_GEMV;
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

        const std::string key = cacheKey(op, inDim, rows, ncol, rep.device);
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
                // a cached schedule that is no longer a candidate (another build) is ignored
                bool legal = false;
                for (uint32_t i = 0; i < n; ++i)
                    legal = legal || (list[i].family == c.schedule.family &&
                                      list[i].rows_in_flight == c.schedule.rows_in_flight &&
                                      list[i].persistent == c.schedule.persistent);
                if (!legal) continue;
                c.pass = true;
                rep.candidates.push_back(c);
                rep.selected = 0;
                rep.fromCache = true;
                install(ctx, rep, baseline != 0);
                return rep;
            }
        }

        SplitMix64 rng{opt.seed};
        std::vector<float> x((size_t)(inDim * ncol));
        for (float &v : x) v = rng.nextSignedUnit();
        std::vector<double> ref((size_t)(rows * ncol), 0.0);
        const int64_t rowBytes = inDim / per * bpb;
        DeviceBuffer dw = r.makeBuffer(weights), dx = r.makeBuffer(x), dy = r.makeBuffer(rows * ncol * 4);
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
                if (op == LEV_OP_Q4_0_GEMV) q4_0RowF64(weights.data() + i * rowBytes, inDim, x.data() + c * inDim, s);
                else q4_kRowF64(weights.data() + i * rowBytes, inDim, x.data() + c * inDim, s);
                ref[(size_t)(c * rows + i)] = s;
            }

        auto launch = [&]() {
            if (op == LEV_OP_Q4_K_GEMV_Q8)
                return lev_hip_q4_k_gemv_q8(ctx, dw.contents(), weights.size(), 0,
                                            static_cast<const int8_t *>(dxq.contents()), dxs.floats(), x.size(),
                                            dy.floats(), (size_t)(rows * ncol), (uint32_t)inDim, (uint32_t)rows,
                                            (uint32_t)ncol);
            if (op == LEV_OP_Q4_0_GEMV)
                return lev_hip_q4_0_gemv(ctx, dw.contents(), weights.size(), 0, dx.floats(), (size_t)inDim,
                                         dy.floats(), (size_t)rows, (uint32_t)inDim, (uint32_t)rows);
            return lev_hip_q4_k_gemv_ncol(ctx, dw.contents(), weights.size(), 0, dx.floats(), x.size(), nullptr,
                                          0.f, dy.floats(), (size_t)(rows * ncol), (uint32_t)inDim, (uint32_t)rows,
                                          (uint32_t)ncol);
        };
        for (uint32_t i = 0; i < n; ++i) {
            ForgeCandidate c;
            c.schedule = list[i];
            check(ctx, lev_hip_forge_select(ctx, (uint32_t)inDim, (uint32_t)rows, (uint32_t)ncol, &list[i]));
            // poison the output so that a candidate that writes nothing cannot pass on the previous one's result
            std::vector<float> poison((size_t)(rows * ncol), NAN);
            check(ctx, lev_hip_buf_upload(ctx, dy.contents(), poison.data(), poison.size() * 4));
            check(ctx, launch());
            check(ctx, lev_hip_sync(ctx));
            c.maxRelErr = maxRelErr(r.read<float>(dy, (size_t)(rows * ncol)), ref);
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
            std::sort(samples.begin(), samples.end());
            c.medianUs = samples.empty() ? 0 : samples[samples.size() / 2];
            rep.candidates.push_back(c);
        }

        // baseline must pass; the fastest passing candidate wins if it beats the baseline by more than the margin
        rep.selected = -1;
        if (!rep.candidates.empty() && rep.candidates[0].pass) {
            rep.selected = 0;
            size_t best = 0;
            for (size_t i = 1; i < rep.candidates.size(); ++i)
                if (rep.candidates[i].pass && rep.candidates[i].medianUs < rep.candidates[best].medianUs) best = i;
            if (best != 0 && rep.candidates[best].medianUs < rep.candidates[0].medianUs * (1.0 - opt.margin))
                rep.selected = (int)best;
        }
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

}  // namespace leviathan

// Parity tests of the C++ host mirror (leviathan_amd/host/leviathan_hip.hpp)
// against the CPU oracle, written the way the reference's own Swift tests
// exercise the same operators (Tests/.../main.swift; line numbers per case).
//
// Needs a GPU.  Prints one "ok <case>" line per case, "FAIL ..." and a
// non-zero exit status otherwise.  `--list` prints the case names and exits
// without touching the device.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "leviathan_hip.hpp"
#include "leviathan_forge.hpp"

extern "C" {
#include "lev_oracle.h"
}

using namespace leviathan;

namespace {

int g_failures = 0;

#define EXPECT(cond)                                                              \
    do {                                                                          \
        if (!(cond)) {                                                            \
            std::printf("FAIL %s:%d: %s\n", __FILE__, __LINE__, #cond);           \
            std::fflush(stdout);                                                  \
            ++g_failures;                                                         \
        }                                                                         \
    } while (0)

template <typename E, typename F>
bool throws_q4(E code, F &&fn) {
    try {
        fn();
    } catch (const Q4Exception &e) {
        return e.code == code;
    } catch (...) {
        return false;
    }
    return false;
}

template <typename F>
bool throws_geometry(F &&fn) {
    try {
        fn();
    } catch (const Gemma4Error &e) {
        return e.kind == Gemma4Error::badTensorGeometry;
    } catch (...) {
        return false;
    }
    return false;
}

double rel_err(const std::vector<float> &got, const std::vector<double> &ref) {
    return levo_max_rel_err(got.data(), got.size(), ref.data(), ref.size());
}

// ---- standalone backends ----------------------------------------------------

// main.swift:727-737: two rows of one block, d = +1 and d = -1, all codes 0.
void q4_backend_2x32() {
    std::vector<uint8_t> w = {0x00, 0x3C};
    w.insert(w.end(), 16, 0);
    w.push_back(0x00);
    w.push_back(0xBC);
    w.insert(w.end(), 16, 0);
    std::vector<float> x(32);
    levo_fill_uniform(7, x.data(), 32);
    float sum = 0.f;
    for (float v : x) sum += v;
    auto [y, ev] = Q4HipBackend::matvecReporting(w, 2, 32, x);
    EXPECT(y.size() == 2);
    EXPECT(std::fabs(y[0] - (-8.f * sum)) < 1e-3f);
    EXPECT(std::fabs(y[1] - (8.f * sum)) < 1e-3f);
    EXPECT(ev.outDim == 2 && ev.inDim == 32);
    EXPECT(!ev.deviceName.empty());
    EXPECT(ev.commandStatus == "completed");
}

// main.swift:5106-5117: codes l | (16+l)<<4 against ones gives -16 exactly.
void q4_backend_minus_16() {
    std::vector<uint8_t> w = {0x00, 0x3C};
    for (int l = 0; l < 16; ++l) w.push_back((uint8_t)((l | ((16 + l) << 4)) & 0xFF));
    std::vector<float> x(32, 1.f);
    EXPECT(Q4HipBackend::matvec(w, 1, 32, x)[0] == -16.f);
}

// main.swift:778-796 and Q4.swift:168-196: every guard fires before the device is used.
void q4_backend_guards() {
    std::vector<uint8_t> none;
    std::vector<float> nox;
    EXPECT(throws_q4(Q4Error::badDimensions, [&] { Q4HipBackend::matvecReporting(none, 8, 33, nox); }));
    EXPECT(throws_q4(Q4Error::badDimensions, [&] { Q4HipBackend::matvecReporting(none, 8, 32, nox); }));
    EXPECT(throws_q4(Q4Error::badDimensions, [&] { Q4HipBackend::matvecReporting(none, 0, 32, nox); }));
    std::vector<uint8_t> w(8 * 18, 0);
    std::vector<float> three(3, 0.f);
    EXPECT(throws_q4(Q4Error::wrongInputCount, [&] { Q4HipBackend::matvecReporting(w, 8, 32, three); }));
    std::vector<float> bad(32, 0.f);
    bad[5] = NAN;
    EXPECT(throws_q4(Q4Error::nonFiniteInput, [&] { Q4HipBackend::matvecReporting(w, 8, 32, bad); }));
    bad[5] = INFINITY;
    EXPECT(throws_q4(Q4Error::nonFiniteInput, [&] { Q4HipBackend::matvecReporting(w, 8, 32, bad); }));
}

// main.swift:1091-1120: the hand-computed Q6_K row, -315 exactly.
void q6_backend_minus_315() {
    std::vector<uint8_t> b(210, 0);
    b[208] = 0x00; b[209] = 0x3C;
    b[192] = 3; b[193] = 0xFD; b[196] = 2; b[200] = 3; b[204] = 2;
    b[0] = 0x21; b[128] = 0x03; b[64] = 0x21; b[160] = 0x01;
    std::vector<float> x(256, 0.f);
    x[0] = 1; x[16] = -1; x[64] = 2; x[128] = -2; x[192] = 4;
    auto [y, ev] = Q6HipBackend::matvecReporting(b, 1, 256, x);
    EXPECT(y.size() == 1 && y[0] == -315.f);
    EXPECT(ev.inDim == 256);
    std::vector<float> shortx(255, 0.f);
    EXPECT(throws_q4(Q4Error::wrongInputCount, [&] { Q6HipBackend::matvecReporting(b, 1, 256, shortx); }));
    EXPECT(throws_q4(Q4Error::badDimensions, [&] { Q6HipBackend::matvecReporting(b, 1, 128, x); }));
}

// Seeded 64x512 against the FP64 oracle, gate 1e-4 (Q4Lowering.swift:887-937).
void q4_backend_seeded() {
    const int rows = 64, cols = 512;
    std::vector<uint8_t> w((size_t)rows * cols / 32 * 18);
    levo_synth_q4_0(21, 0.02f, w.data(), w.size() / 18);
    std::vector<float> x(cols);
    levo_fill_uniform(22, x.data(), cols);
    std::vector<double> ref(rows);
    EXPECT(levo_q4_0_matvec_f64(w.data(), w.size(), rows, cols, x.data(), cols, ref.data()) == 0);
    EXPECT(rel_err(Q4HipBackend::matvec(w, rows, cols, x), ref) < 1e-4);
}

// ---- runner operators --------------------------------------------------------

struct Model {
    // one weight buffer: a Q4_0 matrix, a Q6_K matrix, an F32 norm weight, an
    // F32 router and the expert tensors of layer 0, at 256-byte aligned offsets
    static constexpr int hidden = 256, inter = 128, experts = 8, topK = 2, vocab = 96;
    static constexpr int sharedInter = 192;   // a multiple of 64: the up half of gate|up starts 256-byte aligned
    std::vector<uint8_t> bytes;
    std::map<std::string, TensorRef> table;
    MoEBinding binding;
    int64_t gu_slice, dn_slice;

    int64_t add(const std::string &name, GGMLTensorType t, int64_t inDim, int64_t outDim, int64_t nexp,
                const std::function<void(uint8_t *, size_t)> &fill) {
        size_t start = (bytes.size() + 255) & ~(size_t)255;
        size_t n = (size_t)(inDim / elementsPerBlock(t)) * bytesPerBlock(t) * outDim * nexp;
        bytes.resize(start + n);
        fill(bytes.data() + start, n);
        TensorRef r;
        r.type = t; r.offset = (int64_t)start; r.end = (int64_t)(start + n);
        r.inDim = inDim; r.outDim = outDim; r.experts = nexp;
        table[name] = r;
        return (int64_t)start;
    }

    Model() {
        add("blk.0.attn_q.weight", GGMLTensorType::q4_0, hidden, hidden, 1,
            [](uint8_t *p, size_t n) { levo_synth_q4_0(31, 0.02f, p, n / 18); });
        add("output.weight", GGMLTensorType::q6_K, hidden, vocab, 1,
            [](uint8_t *p, size_t n) { levo_synth_q6_k(32, 0.01f, p, n / 210); });
        add("blk.0.ffn_norm.weight", GGMLTensorType::float32, hidden, 1, 1,
            [](uint8_t *p, size_t n) { levo_fill_normal(33, 1.f, 0.1f, reinterpret_cast<float *>(p), n / 4); });
        add("blk.0.ffn_gate_inp.weight", GGMLTensorType::float32, hidden, experts, 1,
            [](uint8_t *p, size_t n) { levo_fill_normal(34, 0.f, 0.02f, reinterpret_cast<float *>(p), n / 4); });
        add("blk.0.ffn_up.weight", GGMLTensorType::q4_K, hidden, 64, 1,
            [](uint8_t *p, size_t n) { levo_synth_q4_k(37, 0.01f, p, n / 144); });
        // the shared expert of layer 1 (Gemma4.swift:3742-3773)
        add("blk.1.ffn_norm.weight", GGMLTensorType::float32, hidden, 1, 1,
            [](uint8_t *p, size_t n) { levo_fill_normal(61, 1.f, 0.1f, reinterpret_cast<float *>(p), n / 4); });
        add("blk.1.post_ffw_norm_1.weight", GGMLTensorType::float32, hidden, 1, 1,
            [](uint8_t *p, size_t n) { levo_fill_normal(62, 1.f, 0.1f, reinterpret_cast<float *>(p), n / 4); });
        add("blk.1.ffn_gate.weight", GGMLTensorType::q4_0, hidden, sharedInter, 1,
            [](uint8_t *p, size_t n) { levo_synth_q4_0(63, 0.02f, p, n / 18); });
        add("blk.1.ffn_up.weight", GGMLTensorType::q4_0, hidden, sharedInter, 1,
            [](uint8_t *p, size_t n) { levo_synth_q4_0(64, 0.02f, p, n / 18); });
        add("blk.1.ffn_down.weight", GGMLTensorType::q4_0, sharedInter, hidden, 1,
            [](uint8_t *p, size_t n) { levo_synth_q4_0(65, 0.02f, p, n / 18); });
        // fused gate|up [2I, H] per expert, as the reference stores it
        int64_t gu = add("blk.0.ffn_gate_up_exps.weight", GGMLTensorType::q4_0, hidden, 2 * inter, experts,
                         [](uint8_t *p, size_t n) { levo_synth_q4_0(35, 0.02f, p, n / 18); });
        int64_t dn = add("blk.0.ffn_down_exps.weight", GGMLTensorType::q4_0, inter, hidden, experts,
                         [](uint8_t *p, size_t n) { levo_synth_q4_0(36, 0.02f, p, n / 18); });
        gu_slice = (int64_t)2 * inter * (hidden / 32) * 18;
        dn_slice = (int64_t)hidden * (inter / 32) * 18;
        binding.gateOffset = gu;
        binding.upOffset = gu + gu_slice / 2;
        binding.downOffset = dn;
        binding.gateStride = binding.upStride = gu_slice;
        binding.downStride = dn_slice;
        binding.hidden = hidden;
        binding.expertIntermediate = inter;
        binding.experts = experts;
        binding.topK = topK;
    }
    const uint8_t *at(const std::string &name) const { return bytes.data() + table.at(name).offset; }
};

void runner_matvec(Runner &r, const Model &m) {
    const int H = Model::hidden;
    std::vector<float> x(H);
    levo_fill_normal(41, 0.f, 1.f, x.data(), H);
    DeviceBuffer dx = r.makeBuffer(x), dy = r.makeBuffer((int64_t)H * 4 + 256);
    r.matvec("blk.0.attn_q.weight", dx, H, dy, H + 64);
    std::vector<double> ref(H);
    const TensorRef &t = m.table.at("blk.0.attn_q.weight");
    levo_q4_0_matvec_f64(m.at("blk.0.attn_q.weight"), (size_t)(t.end - t.offset), H, H, x.data(), H, ref.data());
    EXPECT(rel_err(r.read<float>(dy, H), ref) < 1e-4);

    // a row range: rows 32.. through extraOffset, written at a shifted output binding
    const int64_t row_bytes = H / 32 * 18;
    r.matvec("blk.0.attn_q.weight", dx, H, dy, H + 64, 32 * row_bytes, 16, 256);
    std::vector<float> all = r.read<float>(dy, H + 64);
    std::vector<float> part(all.begin() + 64, all.begin() + 80);
    std::vector<double> pref(ref.begin() + 32, ref.begin() + 48);
    EXPECT(rel_err(part, pref) < 1e-4);

    // Q6_K head
    DeviceBuffer dl = r.makeBuffer((int64_t)Model::vocab * 4);
    r.matvec("output.weight", dx, H, dl, Model::vocab);
    std::vector<double> lref(Model::vocab);
    const TensorRef &o = m.table.at("output.weight");
    levo_q6_k_matvec_f64(m.at("output.weight"), (size_t)(o.end - o.offset), Model::vocab, H, x.data(), H,
                         lref.data());
    EXPECT(rel_err(r.read<float>(dl, Model::vocab), lref) < 1e-4);

    // guards of Gemma4.swift:2588-2627, each before any launch
    EXPECT(throws_geometry([&] { r.matvec("missing.weight", dx, H, dy, H); }));
    EXPECT(throws_geometry([&] { r.matvec("blk.0.attn_q.weight", dx, H - 1, dy, H); }));          // xCount
    EXPECT(throws_geometry([&] { r.matvec("blk.0.attn_q.weight", dx, H, dy, H - 1); }));          // yCapacity
    EXPECT(throws_geometry([&] { r.matvec("blk.0.attn_q.weight", dx, H, dy, H, 0, std::nullopt, 4); }));  // y offset % 256
    EXPECT(throws_geometry([&] { r.matvec("blk.0.attn_q.weight", dx, H, dy, H, row_bytes, H); }));       // beyond extent
    EXPECT(throws_geometry([&] { r.matvec("blk.0.attn_q.weight", dx, H, dy, H, -18); }));         // before the tensor
    EXPECT(throws_geometry([&] { r.matvec("blk.0.attn_q.weight", dx, H, dy, H, 0, 0); }));        // zero rows
    r.flushOpenSegment();   // nothing failed on the device
}

// Int8-activation decode path: Builder::norm_quant then Builder::matvec
// (rust/crates/lev-model/src/gpu.rs:295-370), gated as vk_q8 does
// (lev-cli/src/main.rs:1788-1868): codes bit-exact with quantize_q8 of the CPU
// rmsnorm, product within 1e-4 of the f64 oracle on those codes.
void runner_int8_path(Runner &r, const Model &m) {
    const int H = Model::hidden, NB = 2, ROWS = 64;
    std::vector<float> x((size_t)NB * H), delta((size_t)NB * H);
    levo_fill_normal(71, 0.f, 1.f, x.data(), x.size());
    levo_fill_normal(72, 0.f, 0.5f, delta.data(), delta.size());
    DeviceBuffer dx = r.makeBuffer(x), dd = r.makeBuffer(delta);
    DeviceBuffer xq = r.makeBuffer((int64_t)NB * H), xs = r.makeBuffer((int64_t)NB * H / 32 * 8);
    DeviceBuffer dyn = r.makeBuffer((int64_t)NB * H * 4), dy = r.makeBuffer((int64_t)NB * ROWS * 4);
    r.normQuant(dx, H, NB, std::string("blk.0.ffn_norm.weight"), xq, xs, &dd, &dyn);
    r.matvecQ8("blk.0.ffn_up.weight", xq, xs, NB, dy);
    std::vector<float> xsum = r.read<float>(dx, x.size()), yn = r.read<float>(dyn, x.size());
    std::vector<int8_t> q = r.read<int8_t>(xq, x.size());
    std::vector<float> pairs = r.read<float>(xs, (size_t)NB * H / 32 * 2), y = r.read<float>(dy, (size_t)NB * ROWS);
    const float *gain = reinterpret_cast<const float *>(m.at("blk.0.ffn_norm.weight"));
    const TensorRef &t = m.table.at("blk.0.ffn_up.weight");
    for (int c = 0; c < NB; ++c) {
        std::vector<float> sum(H), want(H), wd(H / 32), ws(H / 32), xd(H);
        std::vector<int8_t> wq(H);
        for (int i = 0; i < H; ++i) sum[i] = x[(size_t)c * H + i] + delta[(size_t)c * H + i];
        levo_rmsnorm(sum.data(), gain, 1e-6f, H, want.data());
        EXPECT(levo_quantize_q8(want.data(), H, wq.data(), wd.data(), ws.data()) == 0);
        EXPECT(std::memcmp(xsum.data() + (size_t)c * H, sum.data(), H * 4) == 0);      // x += add, written back
        EXPECT(std::memcmp(yn.data() + (size_t)c * H, want.data(), H * 4) == 0);      // f32 result
        EXPECT(std::memcmp(q.data() + (size_t)c * H, wq.data(), H) == 0);
        for (int g = 0; g < H / 32; ++g) {
            EXPECT(pairs[((size_t)c * (H / 32) + g) * 2] == wd[g]);
            EXPECT(pairs[((size_t)c * (H / 32) + g) * 2 + 1] == ws[g]);
        }
        for (int i = 0; i < H; ++i) xd[i] = (float)wq[i] * wd[i / 32];                 // lev-cpu/src/lib.rs:327
        std::vector<double> ref(ROWS);
        EXPECT(levo_q4_k_matvec_f64(m.at("blk.0.ffn_up.weight"), (size_t)(t.end - t.offset), ROWS, H, xd.data(), H,
                                    ref.data()) == 0);
        std::vector<float> got(y.begin() + (size_t)c * ROWS, y.begin() + (size_t)(c + 1) * ROWS);
        EXPECT(rel_err(got, ref) < 1e-4);
    }
    // the Q6_K head on the same activations
    DeviceBuffer dl = r.makeBuffer((int64_t)NB * Model::vocab * 4);
    r.matvecQ8("output.weight", xq, xs, NB, dl);
    std::vector<float> logits = r.read<float>(dl, (size_t)NB * Model::vocab);
    const TensorRef &o = m.table.at("output.weight");
    for (int c = 0; c < NB; ++c) {
        std::vector<float> xd(H);
        for (int i = 0; i < H; ++i) xd[i] = (float)q[(size_t)c * H + i] * pairs[((size_t)c * (H / 32) + i / 32) * 2];
        std::vector<double> ref(Model::vocab);
        EXPECT(levo_q6_k_matvec_f64(m.at("output.weight"), (size_t)(o.end - o.offset), Model::vocab, H, xd.data(), H,
                                    ref.data()) == 0);
        std::vector<float> got(logits.begin() + (size_t)c * Model::vocab, logits.begin() + (size_t)(c + 1) * Model::vocab);
        EXPECT(rel_err(got, ref) < 1e-4);
    }
    // embedding gather from the same Q4_K tensor used as a [64][256] table: rows 63, 0, 5
    {
        std::vector<uint32_t> tok = {63, 0, 5};
        DeviceBuffer dt = r.makeBuffer(tok), de = r.makeBuffer((int64_t)3 * H * 4);
        r.embed("blk.0.ffn_up.weight", dt, 3, de);
        std::vector<float> e = r.read<float>(de, (size_t)3 * H), want(H);
        for (int c = 0; c < 3; ++c) {
            levo_q4_k_dequant_block_f32(m.at("blk.0.ffn_up.weight") + (size_t)tok[c] * 144, want.data());
            EXPECT(std::memcmp(e.data() + (size_t)c * H, want.data(), H * 4) == 0);
        }
        EXPECT(throws_geometry([&] { r.embed("blk.0.attn_q.weight", dt, 3, de); }));
        EXPECT(throws_geometry([&] { r.embed("blk.0.ffn_up.weight", dt, 4, de); }));
    }
    // a prefix of the rows (matvec_rows), and the guards before any launch
    r.matvecQ8("blk.0.ffn_up.weight", xq, xs, NB, dy, 0, 16);
    std::vector<float> y16 = r.read<float>(dy, (size_t)NB * 16);
    for (int c = 0; c < NB; ++c)
        for (int i = 0; i < 16; ++i) EXPECT(y16[(size_t)c * 16 + i] == y[(size_t)c * ROWS + i]);
    EXPECT(throws_geometry([&] { r.matvecQ8("blk.0.attn_q.weight", xq, xs, NB, dy); }));        // not Q4_K
    EXPECT(throws_geometry([&] { r.matvecQ8("blk.0.ffn_up.weight", xq, xs, NB + 1, dy); }));    // xq too small
    EXPECT(throws_geometry([&] { r.matvecQ8("blk.0.ffn_up.weight", xq, xs, NB, dy, 8); }));     // y too small
    EXPECT(throws_geometry([&] { r.normQuant(dx, H - 32 + 1, 1, std::nullopt, xq, xs); }));     // not a multiple of 32
    EXPECT(throws_geometry([&] { r.normQuant(dx, H, NB + 1, std::nullopt, xq, xs); }));
    EXPECT(throws_geometry([&] { r.normQuant(dx, H, NB, std::string("blk.0.attn_q.weight"), xq, xs); }));
    r.flushOpenSegment();
}

// F32-activation multi-column path: the RMSNorm of Builder::norm_quant fused in front of
// Builder::matvec (rust/crates/lev-model/src/gpu.rs:295-370), every column per one pass over a
// Q4_K tensor or the Q6_K head, gated at 1e-4 against the FP64 product on the CPU rmsnorm.
void runner_f32_columns(Runner &r, const Model &m) {
    const int H = Model::hidden, NB = 3, ROWS = 64;
    std::vector<float> x((size_t)NB * H);
    levo_fill_normal(81, 0.f, 1.f, x.data(), x.size());
    DeviceBuffer dx = r.makeBuffer(x);
    DeviceBuffer dy = r.makeBuffer((int64_t)NB * ROWS * 4), dl = r.makeBuffer((int64_t)NB * Model::vocab * 4);
    const float *gain = reinterpret_cast<const float *>(m.at("blk.0.ffn_norm.weight"));
    const TensorRef &t = m.table.at("blk.0.ffn_up.weight"), &o = m.table.at("output.weight");
    r.matvecCols("blk.0.ffn_up.weight", dx, NB, dy, std::string("blk.0.ffn_norm.weight"));
    r.matvecCols("output.weight", dx, NB, dl, std::string("blk.0.ffn_norm.weight"));
    std::vector<float> y = r.read<float>(dy, (size_t)NB * ROWS), logits = r.read<float>(dl, (size_t)NB * Model::vocab);
    for (int c = 0; c < NB; ++c) {
        std::vector<float> xn(H);
        levo_rmsnorm(x.data() + (size_t)c * H, gain, 1e-6f, H, xn.data());
        std::vector<double> ref(ROWS), lref(Model::vocab);
        EXPECT(levo_q4_k_matvec_f64(m.at("blk.0.ffn_up.weight"), (size_t)(t.end - t.offset), ROWS, H, xn.data(), H,
                                    ref.data()) == 0);
        EXPECT(levo_q6_k_matvec_f64(m.at("output.weight"), (size_t)(o.end - o.offset), Model::vocab, H, xn.data(), H,
                                    lref.data()) == 0);
        EXPECT(rel_err(std::vector<float>(y.begin() + (size_t)c * ROWS, y.begin() + (size_t)(c + 1) * ROWS), ref) < 1e-4);
        EXPECT(rel_err(std::vector<float>(logits.begin() + (size_t)c * Model::vocab,
                                          logits.begin() + (size_t)(c + 1) * Model::vocab), lref) < 1e-4);
    }
    // no gain: the plain product; one column alone gives the same bits as in company
    DeviceBuffer d1 = r.makeBuffer((int64_t)Model::vocab * 4);
    r.matvecCols("output.weight", dx, NB, dl);
    r.matvecCols("output.weight", dx, 1, d1);
    std::vector<float> all = r.read<float>(dl, (size_t)NB * Model::vocab), one = r.read<float>(d1, Model::vocab);
    EXPECT(std::memcmp(all.data(), one.data(), (size_t)Model::vocab * 4) == 0);
    std::vector<double> lref(Model::vocab);
    EXPECT(levo_q6_k_matvec_f64(m.at("output.weight"), (size_t)(o.end - o.offset), Model::vocab, H, x.data(), H,
                                lref.data()) == 0);
    EXPECT(rel_err(one, lref) < 1e-4);
    // and the single-column operator agrees bit for bit
    DeviceBuffer ds = r.makeBuffer((int64_t)Model::vocab * 4);
    r.matvec("output.weight", dx, H, ds, Model::vocab);
    EXPECT(std::memcmp(r.read<float>(ds, Model::vocab).data(), one.data(), (size_t)Model::vocab * 4) == 0);
    // a prefix of the rows, and the guards before any launch
    r.matvecCols("blk.0.ffn_up.weight", dx, NB, dy, std::nullopt, 0, 16);
    EXPECT(throws_geometry([&] { r.matvecCols("blk.0.attn_q.weight", dx, NB, dy); }));                 // Q4_0
    EXPECT(throws_geometry([&] { r.matvecCols("blk.0.ffn_up.weight", dx, NB + 1, dy); }));             // x too small
    EXPECT(throws_geometry([&] { r.matvecCols("blk.0.ffn_up.weight", dx, NB, dy, std::nullopt, 8); })); // y too small
    EXPECT(throws_geometry([&] { r.matvecCols("blk.0.ffn_up.weight", dx, NB, dy, std::string("blk.0.attn_q.weight")); }));
    r.flushOpenSegment();
}

void runner_elementwise(Runner &r, const Model &m) {
    const int H = Model::hidden, V = 3;
    std::vector<float> x((size_t)V * H);
    levo_fill_normal(51, 0.f, 1.f, x.data(), x.size());
    DeviceBuffer dx = r.makeBuffer(x), dy = r.makeBuffer((int64_t)V * H * 4);
    r.rmsnorm(dx, dy, H, V, std::string("blk.0.ffn_norm.weight"));
    std::vector<float> y = r.read<float>(dy, (size_t)V * H);
    const float *gain = reinterpret_cast<const float *>(m.at("blk.0.ffn_norm.weight"));
    for (int v = 0; v < V; ++v) {
        std::vector<double> ref(H);
        levo_rmsnorm_f64(x.data() + (size_t)v * H, gain, 1e-6, H, ref.data());
        std::vector<float> got(y.begin() + (size_t)v * H, y.begin() + (size_t)(v + 1) * H);
        EXPECT(rel_err(got, ref) < 1e-5);
    }
    // lev-model lib.rs:431-435: x = 2, no weight -> 1 (times w = 0.5 there)
    std::vector<float> twos(H, 2.f);
    DeviceBuffer d2 = r.makeBuffer(twos), dn = r.makeBuffer((int64_t)H * 4);
    r.rmsnorm(d2, dn, H, 1, std::nullopt);
    for (float v : r.read<float>(dn, H)) EXPECT(std::fabs(v - 1.f) < 1e-5f);
    EXPECT(throws_geometry([&] { r.rmsnorm(dx, dy, H, V + 1, std::nullopt); }));
    EXPECT(throws_geometry([&] { r.rmsnorm(dx, dy, H / 2, 1, std::string("blk.0.ffn_norm.weight")); }));
    EXPECT(throws_geometry([&] { r.rmsnorm(dx, dy, H, 1, std::string("blk.0.attn_q.weight")); }));

    // geluUp: main.swift:8947-8950 and 6680-6690
    std::vector<float> gu = {1.f, -20.f, 1e30f, -1e30f, 1e-30f, 1e20f, 0.5f, -0.5f,
                             1.f, 3.f, 2.f, 2.f, 2.f, 2.f, 4.f, 4.f};
    DeviceBuffer dgu = r.makeBuffer(gu), dact = r.makeBuffer((int64_t)8 * 4);
    r.geluUp(dgu, dact, 8);
    std::vector<float> act = r.read<float>(dact, 8);
    EXPECT(std::fabs(act[0] - 0.841192f) < 1e-6f);
    EXPECT(act[1] == 0.f || std::fabs(act[1]) < 1e-30f);
    for (int i = 0; i < 8; ++i) {
        EXPECT(std::isfinite(act[i]));
        float want = levo_gelu_up_f32(gu[i], gu[8 + i]);
        EXPECT(std::fabs(act[i] - want) <= 1e-6f * std::fmax(1.f, std::fabs(want)));
    }
    EXPECT(throws_geometry([&] { r.geluUp(dgu, dact, 9); }));

    // axpy: Gemma4.swift:3115-3140
    std::vector<float> a = {1, 2, 3, 4, 5, 6, 7, 8}, b = {10, 20, 30, 40};
    DeviceBuffer da = r.makeBuffer(a), db = r.makeBuffer(b);
    r.axpy(da, db, 0.5f, 4, 16);   // x from element 4
    std::vector<float> got = r.read<float>(db, 4);
    EXPECT(got[0] == 12.5f && got[1] == 23.f && got[2] == 33.5f && got[3] == 44.f);
    EXPECT(throws_geometry([&] { r.axpy(da, db, 1.f, 0); }));
    EXPECT(throws_geometry([&] { r.axpy(da, db, NAN, 4); }));
    EXPECT(throws_geometry([&] { r.axpy(da, db, 1.f, 4, 2); }));     // offset % 4
    EXPECT(throws_geometry([&] { r.axpy(da, db, 1.f, 4, 20); }));    // beyond x
    EXPECT(throws_geometry([&] { r.axpy(da, db, 1.f, 5); }));        // beyond y
}

void runner_moe(Runner &r, const Model &m) {
    const int H = Model::hidden, I = Model::inter, K = Model::topK;
    std::vector<float> x(H);
    levo_fill_normal(61, 0.f, 1.f, x.data(), H);
    DeviceBuffer dx = r.makeBuffer(x), dy = r.makeBuffer((int64_t)H * 4);

    // router: ids bit-exact, weights to 1e-6 (Gemma4.swift:3795-3810)
    auto [topIdx, weights] = r.routeTopK("blk.0.ffn_gate_inp.weight", dx, K);
    std::vector<float> scores(Model::experts);
    levo_f32_matvec(reinterpret_cast<const float *>(m.at("blk.0.ffn_gate_inp.weight")), Model::experts, H,
                    x.data(), scores.data());
    std::vector<int32_t> rid(K);
    std::vector<float> rw(K);
    EXPECT(levo_router_topk(scores.data(), Model::experts, K, nullptr, rid.data(), rw.data()) == 0);
    for (int k = 0; k < K; ++k) {
        EXPECT(topIdx[k] == rid[k]);
        EXPECT(std::fabs(weights[k] - rw[k]) < 1e-6f);
    }

    // routed experts against the FP64 oracle (MoESIMDLowering.swift:986-1030), gate 1e-4
    r.runMoeBatchedRouted(dx, dy, topIdx, weights, m.binding);
    std::vector<float> y = r.read<float>(dy, H);
    const uint8_t *gate = m.bytes.data() + m.binding.gateOffset;
    const uint8_t *up = m.bytes.data() + m.binding.upOffset;
    const uint8_t *down = m.bytes.data() + m.binding.downOffset;
    std::vector<double> yref(H), g((size_t)K * I), u((size_t)K * I), a((size_t)K * I), d((size_t)K * H);
    EXPECT(levo_moe_experts_f64(gate, up, down, (size_t)m.gu_slice, (size_t)m.gu_slice, (size_t)m.dn_slice, H, I,
                                K, rid.data(), rw.data(), x.data(), yref.data(), g.data(), u.data(), a.data(),
                                d.data()) == 0);
    EXPECT(rel_err(y, yref) < 1e-4);

    // the same through the per-slot operators, as forwardLayer's serial loop does
    // (Gemma4.swift:3856-3880): expertMatvec(gate_up) -> geluUp -> expertMatvec(down) -> axpy
    DeviceBuffer dgu = r.makeBuffer((int64_t)2 * I * 4), dact = r.makeBuffer((int64_t)I * 4),
                 ddn = r.makeBuffer((int64_t)H * 4);
    DeviceBuffer dacc = r.makeBuffer(std::vector<float>(H, 0.f));
    for (int k = 0; k < K; ++k) {
        r.expertMatvec("blk.0.ffn_gate_up_exps.weight", 0, topIdx[k], dx, H, dgu, 2 * I);
        r.geluUp(dgu, dact, I);
        r.expertMatvec("blk.0.ffn_down_exps.weight", 0, topIdx[k], dact, I, ddn, H);
        r.axpy(ddn, dacc, weights[k], H);
    }
    std::vector<float> yserial = r.read<float>(dacc, H);
    EXPECT(rel_err(yserial, yref) < 1e-4);
    std::vector<double> yd(y.begin(), y.end());
    EXPECT(rel_err(yserial, yd) < 1e-5);   // the composite and the serial loop agree

    // guards: MoEModelBinding.offsets and Gemma4.swift:2094-2110
    EXPECT(throws_geometry([&] { r.runMoeBatchedRouted(dx, dy, {0, 0}, weights, m.binding); }));
    EXPECT(throws_geometry([&] { r.runMoeBatchedRouted(dx, dy, {0, Model::experts}, weights, m.binding); }));
    EXPECT(throws_geometry([&] { r.runMoeBatchedRouted(dx, dy, {0, -1}, weights, m.binding); }));
    EXPECT(throws_geometry([&] { r.runMoeBatchedRouted(dx, dy, {0}, weights, m.binding); }));
    EXPECT(throws_geometry([&] { r.runMoeBatchedRouted(dx, dy, topIdx, {0.5f}, m.binding); }));
    EXPECT(throws_geometry([&] { r.runMoeBatchedRouted(dx, dy, topIdx, {0.5f, NAN}, m.binding); }));
    EXPECT(throws_geometry([&] { r.runMoeBatchedRouted(dx, dx, topIdx, weights, m.binding); }));
    EXPECT(throws_geometry([&] { r.expertMatvec("blk.0.attn_q.weight", 0, 0, dx, H, dgu, 2 * I); }));
    EXPECT(throws_geometry([&] { r.expertMatvec("blk.0.ffn_gate_up_exps.weight", 1, 0, dx, H, dgu, 2 * I); }));
    EXPECT(throws_geometry([&] { r.expertMatvec("blk.0.ffn_gate_up_exps.weight", 0, Model::experts, dx, H, dgu, 2 * I); }));
    EXPECT(throws_geometry([&] { r.expertMatvec("blk.0.ffn_gate_up_exps.weight", 0, 0, dx, H, dgu, 2 * I - 1); }));
    r.flushOpenSegment();
}

// main.swift:8925-8946: 32/32/top-1, gate 16, up 2, act 32, down 512 -- exact.
void runner_moe_hand_computed(Runner &) {
    auto rows = [](uint8_t lo, uint8_t hi, uint8_t q) {
        std::vector<uint8_t> out;
        for (int r = 0; r < 32; ++r) {
            out.push_back(lo);
            out.push_back(hi);
            out.insert(out.end(), 16, q);
        }
        return out;
    };
    std::vector<uint8_t> bytes = rows(0x00, 0x3C, 0x98), up = rows(0x00, 0x30, 0x98), down = rows(0x00, 0x38, 0x99);
    MoEBinding b;
    b.gateOffset = 0;
    b.upOffset = (int64_t)bytes.size();
    bytes.insert(bytes.end(), up.begin(), up.end());
    b.downOffset = (int64_t)bytes.size();
    bytes.insert(bytes.end(), down.begin(), down.end());
    b.gateStride = b.upStride = b.downStride = 32 * 18;
    b.hidden = 32; b.expertIntermediate = 32; b.experts = 1; b.topK = 1;
    Runner r2;
    r2.bindWeights(bytes, {});
    DeviceBuffer dx = r2.makeBuffer(std::vector<float>(32, 1.f)), dy = r2.makeBuffer((int64_t)32 * 4);
    r2.runMoeBatchedRouted(dx, dy, {0}, {1.0f}, b);
    for (float v : r2.read<float>(dy, 32)) EXPECT(v == 512.f);
    r2.runMoeBatchedRouted(dx, dy, {0}, {0.5f}, b);
    for (float v : r2.read<float>(dy, 32)) EXPECT(v == 256.f);
}

struct Case {
    const char *name;
    std::function<void()> run;
};

}  // namespace

// ---- model file -> resident buffer -> kernels ----------------------------------
// The Model's tensors written as a GGUF v3 file (gemma4 metadata, 32-byte
// alignment), read back through GGUFFile / MoEModelBinding / Runner::bindGGUF:
// the same operators must give the same bits as on the memory-bound weights.
static void put_u32(std::vector<uint8_t> &o, uint32_t v) { o.insert(o.end(), (uint8_t *)&v, (uint8_t *)&v + 4); }
static void put_u64(std::vector<uint8_t> &o, uint64_t v) { o.insert(o.end(), (uint8_t *)&v, (uint8_t *)&v + 8); }
static void put_str(std::vector<uint8_t> &o, const std::string &s) {
    put_u64(o, s.size());
    o.insert(o.end(), s.begin(), s.end());
}

std::string write_model_gguf(const Model &m) {
    std::vector<uint8_t> o = {'G', 'G', 'U', 'F'};
    put_u32(o, 3);
    put_u64(o, m.table.size());
    put_u64(o, 6);
    put_str(o, "general.architecture"); put_u32(o, 8); put_str(o, "gemma4");
    const std::pair<const char *, uint32_t> ints[] = {
        {"gemma4.block_count", 1}, {"gemma4.expert_count", Model::experts}, {"gemma4.expert_used_count", Model::topK},
        {"gemma4.embedding_length", Model::hidden}, {"gemma4.expert_feed_forward_length", Model::inter}};
    for (auto &kv : ints) {
        put_str(o, kv.first);
        put_u32(o, 4);
        put_u32(o, kv.second);
    }
    uint64_t off = 0;
    std::vector<std::pair<const TensorRef *, uint64_t>> placed;
    for (auto &kv : m.table) {
        const TensorRef &t = kv.second;
        put_str(o, kv.first);
        const bool three = t.experts > 1, one = t.outDim == 1 && !three;
        put_u32(o, three ? 3 : one ? 1 : 2);
        put_u64(o, (uint64_t)t.inDim);
        if (!one) put_u64(o, (uint64_t)t.outDim);
        if (three) put_u64(o, (uint64_t)t.experts);
        put_u32(o, (uint32_t)t.type);
        off = (off + 31) / 32 * 32;
        put_u64(o, off);
        placed.push_back({&t, off});
        off += (uint64_t)(t.end - t.offset);
    }
    while (o.size() % 32) o.push_back(0);
    const size_t data0 = o.size();
    o.resize(data0 + off);
    for (auto &pl : placed)
        std::memcpy(o.data() + data0 + pl.second, m.bytes.data() + pl.first->offset, (size_t)(pl.first->end - pl.first->offset));
    char path[] = "/tmp/lev_host_parity_XXXXXX";
    const int fd = mkstemp(path);
    EXPECT(fd >= 0);
    FILE *f = fdopen(fd, "wb");
    EXPECT(f && std::fwrite(o.data(), 1, o.size(), f) == o.size());
    if (f) std::fclose(f);
    return path;
}

void runner_gguf_file(Runner &mem, const Model &m) {
    const std::string path = write_model_gguf(m);
    Runner r(0);
    GGUFFile g = r.bindGGUF(path);
    EXPECT(g.version == 3 && g.tensors.size() == m.table.size() && g.alignment == 32);
    MoEModelBinding mb = MoEModelBinding::bind(g);
    EXPECT(mb.layerCount == 1 && mb.expertCount == Model::experts && mb.topK == Model::topK);
    EXPECT(mb.guStride == m.gu_slice && mb.dnStride == m.dn_slice);
    const MoEBinding bind = Runner::moeBinding(mb, 0);
    std::remove(path.c_str());

    const int H = Model::hidden, K = Model::topK;
    std::vector<float> x(H);
    levo_fill_normal(91, 0.f, 1.f, x.data(), H);
    auto both = [&](auto &&fn) {   // the file-bound and the memory-bound runner, same operator
        std::vector<float> a = fn(r), b = fn(mem);
        EXPECT(a.size() == b.size() && std::memcmp(a.data(), b.data(), a.size() * 4) == 0);
        return a;
    };
    std::vector<float> y = both([&](Runner &rr) {
        DeviceBuffer dx = rr.makeBuffer(x), dy = rr.makeBuffer((int64_t)H * 4);
        rr.matvec("blk.0.attn_q.weight", dx, H, dy, H);
        return rr.read<float>(dy, H);
    });
    std::vector<double> ref(H);
    const TensorRef &t = m.table.at("blk.0.attn_q.weight");
    levo_q4_0_matvec_f64(m.at("blk.0.attn_q.weight"), (size_t)(t.end - t.offset), H, H, x.data(), H, ref.data());
    EXPECT(rel_err(y, ref) < 1e-4);
    both([&](Runner &rr) {
        DeviceBuffer dx = rr.makeBuffer(x), dl = rr.makeBuffer((int64_t)Model::vocab * 4);
        rr.matvec("output.weight", dx, H, dl, Model::vocab);
        return rr.read<float>(dl, Model::vocab);
    });
    // the MoE block through the binding taken from the file
    std::vector<int32_t> ids;
    std::vector<float> wts;
    std::vector<float> ym = both([&](Runner &rr) {
        DeviceBuffer dx = rr.makeBuffer(x), dy = rr.makeBuffer((int64_t)H * 4);
        auto [topIdx, weights] = rr.routeTopK("blk.0.ffn_gate_inp.weight", dx, K);
        ids.assign(topIdx.begin(), topIdx.end());
        wts = weights;
        rr.runMoeBatchedRouted(dx, dy, topIdx, weights, &rr == &r ? bind : m.binding);
        return rr.read<float>(dy, H);
    });
    std::vector<double> yref(H), gg((size_t)K * Model::inter), uu(gg.size()), aa(gg.size()), dd((size_t)K * H);
    EXPECT(levo_moe_experts_f64(m.bytes.data() + m.binding.gateOffset, m.bytes.data() + m.binding.upOffset,
                                m.bytes.data() + m.binding.downOffset, (size_t)m.gu_slice, (size_t)m.gu_slice,
                                (size_t)m.dn_slice, H, Model::inter, K, ids.data(), wts.data(), x.data(), yref.data(),
                                gg.data(), uu.data(), aa.data(), dd.data()) == 0);
    EXPECT(rel_err(ym, yref) < 1e-4);
    // slice offsets of a route: exactly the operator's own addressing
    std::vector<uint64_t> gu, dn;
    mb.offsets(0, {Model::experts - 1, 0}, gu, dn);
    EXPECT(gu[0] == (uint64_t)(bind.gateOffset + (Model::experts - 1) * bind.gateStride) && gu[1] == (uint64_t)bind.gateOffset);
    EXPECT(dn[1] == (uint64_t)bind.downOffset);
    bool threw = false;
    try {
        mb.offsets(0, {0, 0}, gu, dn);
    } catch (const GGUFError &) {
        threw = true;
    }
    EXPECT(threw);
}


// Forge loop (lev-cli/src/main.rs:1941-2024): baseline first, every candidate
// gated against the FP64 oracle, the 2 % rule, the cache, and a gate nobody passes.
void forge_matvec(Runner &r) {
    struct Shape { GGMLTensorType type; int rows, cols, ncol; };
    const Shape shapes[] = {{GGMLTensorType::q4_0, 512, 4096, 1}, {GGMLTensorType::q4_0, 300, 2048, 1},
                            {GGMLTensorType::q4_0, 64, 256, 1}, {GGMLTensorType::q4_K, 256, 1024, 1},
                            {GGMLTensorType::q4_K, 128, 512, 3}, {GGMLTensorType::q6_K, 200, 4096, 1},
                            {GGMLTensorType::q6_K, 96, 1024, 1}};
    const std::string cache = "/tmp/leviathan_forge_test_cache.txt";
    std::remove(cache.c_str());
    for (const Shape &sh : shapes) {
        const bool q40 = sh.type == GGMLTensorType::q4_0, q6 = sh.type == GGMLTensorType::q6_K;
        std::vector<uint8_t> w((size_t)sh.rows * sh.cols / (q40 ? 32 : 256) * (q40 ? 18 : q6 ? 210 : 144));
        if (q40) levo_synth_q4_0(51, 0.02f, w.data(), w.size() / 18);
        else if (q6) levo_synth_q6_k(54, 0.01f, w.data(), w.size() / 210);
        else levo_synth_q4_k(52, 0.01f, w.data(), w.size() / 144);
        ForgeOptions opt;
        opt.launchesPerSample = 5;
        opt.cachePath = cache;
        opt.rotateBytes = 8 << 20;
        ForgeReport rep = MatvecForge::forge(r, sh.type, w, sh.rows, sh.cols, sh.ncol, opt);
        EXPECT(!rep.fromCache);
        EXPECT(!rep.candidates.empty());
        EXPECT(q40 || q6 || rep.candidates.size() == 2);                 // matrix-core and vector-ALU kernel
        // matrix-core kernels (a wave per superblock column for these rows of at most sixteen superblocks, then
        // the several-column kernel with its built-in waves per row group, then 2 and 4 where they differ), dot4
        // kernel (two waves, one wave a row), f64-sum kernel
        EXPECT(!q6 || rep.candidates.size() == (sh.cols == 4096 ? 7u : 5u));
        EXPECT(!q6 || (rep.candidates[0].schedule.family == 2u && rep.candidates[0].schedule.rows_in_flight == 0u));
        // matrix-core kernel (two grids) first, then the vector-ALU kernels: 3 depths x 2 grids, or one for narrow rows
        EXPECT(!q40 || sh.cols < 1024 || rep.candidates.size() == 8);
        EXPECT(!q40 || sh.cols >= 1024 || rep.candidates.size() == 3);
        EXPECT(!q40 || rep.candidates[0].schedule.family == 1u);
        for (const ForgeCandidate &c : rep.candidates) {
            EXPECT(c.pass);
            EXPECT(c.maxRelErr >= 0 && c.maxRelErr < 1e-4);
            EXPECT(c.medianUs > 0);
        }
        EXPECT(rep.selected >= 0 && rep.selected < (int)rep.candidates.size());
        if (rep.selected > 0)
            EXPECT(rep.candidates[(size_t)rep.selected].medianUs < 0.98 * rep.candidates[0].medianUs);
        // the oracle inside the forge agrees with the test oracle on the same inputs
        std::vector<float> x((size_t)sh.cols);
        levo_fill_signed_unit(0x4C455649ull, x.data(), x.size());
        std::vector<double> ref((size_t)sh.rows), mine((size_t)sh.rows, 0.0);
        if (q40) levo_q4_0_matvec_f64(w.data(), w.size(), sh.rows, sh.cols, x.data(), sh.cols, ref.data());
        else if (q6) levo_q6_k_matvec_f64(w.data(), w.size(), sh.rows, sh.cols, x.data(), sh.cols, ref.data());
        else levo_q4_k_matvec_f64(w.data(), w.size(), sh.rows, sh.cols, x.data(), sh.cols, ref.data());
        const size_t row_bytes = w.size() / (size_t)sh.rows;
        double worst = 0;
        for (int i = 0; i < sh.rows; ++i) {
            if (q40) forge_detail::q4_0RowF64(w.data() + i * row_bytes, sh.cols, x.data(), mine[(size_t)i]);
            else if (q6) forge_detail::q6_kRowF64(w.data() + i * row_bytes, sh.cols, x.data(), mine[(size_t)i]);
            else forge_detail::q4_kRowF64(w.data() + i * row_bytes, sh.cols, x.data(), mine[(size_t)i]);
            worst = std::max(worst, std::fabs(mine[(size_t)i] - ref[(size_t)i]) / std::max(1.0, std::fabs(ref[(size_t)i])));
        }
        EXPECT(worst < 1e-12);
        // second call: served from the cache, same schedule
        ForgeReport again = MatvecForge::forge(r, sh.type, w, sh.rows, sh.cols, sh.ncol, opt);
        EXPECT(again.fromCache && again.candidates.size() == 1);
        const lev_schedule &a = again.candidates[0].schedule, &b = rep.candidates[(size_t)rep.selected].schedule;
        EXPECT(a.family == b.family && a.rows_in_flight == b.rows_in_flight && a.persistent == b.persistent);
        // a gate nobody passes selects nothing and leaves the built-in choice
        ForgeOptions strict;
        strict.launchesPerSample = 1;
        strict.timed = 1;
        strict.warm = 0;
        strict.gate = 0.0;
        ForgeReport none = MatvecForge::forge(r, sh.type, w, sh.rows, sh.cols, sh.ncol, strict);
        EXPECT(none.selected == -1);
    }
    // a cached selection is gated again before it is installed: with a gate nobody passes the
    // cache line is skipped and the candidates are run (and rejected) afresh
    {
        std::vector<uint8_t> w((size_t)300 * 2048 / 32 * 18);
        levo_synth_q4_0(51, 0.02f, w.data(), w.size() / 18);
        ForgeOptions strict;
        strict.launchesPerSample = 1;
        strict.timed = 1;
        strict.warm = 0;
        strict.gate = 0.0;
        strict.cachePath = cache;
        ForgeReport none = MatvecForge::forge(r, GGMLTensorType::q4_0, w, 300, 2048, 1, strict);
        EXPECT(!none.fromCache && none.selected == -1);
    }
    std::remove(cache.c_str());
    // the int8-activation GEMV: dot4 kernel and integer matrix-core kernel, gated on the device's own codes
    for (int ncol : {1, 12}) {
        const int rows = 192, cols = 1024;
        std::vector<uint8_t> w((size_t)rows * cols / 256 * 144);
        levo_synth_q4_k(53, 0.01f, w.data(), w.size() / 144);
        ForgeOptions opt;
        opt.launchesPerSample = 5;
        opt.int8Activations = true;
        ForgeReport rep = MatvecForge::forge(r, GGMLTensorType::q4_K, w, rows, cols, ncol, opt);
        EXPECT(rep.op == LEV_OP_Q4_K_GEMV_Q8 && rep.candidates.size() == 2);
        EXPECT(rep.candidates[0].schedule.family == 1u);   // the built-in choice first: matrix cores for rows up to 4096 wide
        for (const ForgeCandidate &c : rep.candidates) EXPECT(c.pass && c.maxRelErr < 1e-4);
        EXPECT(rep.selected >= 0);
    }
    // the Q6_K head over int8 activations: the matrix-core kernel, then the dot4 kernel's grids and column passes
    for (int ncol : {1, 4}) {
        const int rows = 160, cols = 1024;
        std::vector<uint8_t> w((size_t)rows * cols / 256 * 210);
        levo_synth_q6_k(55, 0.01f, w.data(), w.size() / 210);
        ForgeOptions opt;
        opt.launchesPerSample = 5;
        opt.int8Activations = true;
        opt.rotateBytes = 8 << 20;
        ForgeReport rep = MatvecForge::forge(r, GGMLTensorType::q6_K, w, rows, cols, ncol, opt);
        EXPECT(rep.op == LEV_OP_Q6_K_GEMV_Q8 && rep.candidates.size() == (ncol == 1 ? 3u : 4u));
        EXPECT(rep.candidates[0].schedule.family == 1u);
        for (const ForgeCandidate &c : rep.candidates) EXPECT(c.pass && c.maxRelErr < 1e-4 && c.medianUs > 0);
        EXPECT(rep.selected >= 0);
    }
    // misuse of the selection ABI
    lev_ctx *ctx = r.context();
    lev_schedule bogus{LEV_OP_Q4_0_GEMV, 0u, 3u, 0u};
    EXPECT(lev_hip_forge_select(ctx, 4096, 512, 1, &bogus) == LEV_ERR_INVALID_ARGUMENT);
    lev_schedule wrong_op{7u, 0u, 1u, 0u};
    EXPECT(lev_hip_forge_select(ctx, 4096, 512, 1, &wrong_op) == LEV_ERR_INVALID_ARGUMENT);
    uint32_t n = 0;
    EXPECT(lev_hip_forge_candidates(ctx, LEV_OP_Q4_K_GEMV, 100, 8, 1, nullptr, 0, &n) == LEV_ERR_BAD_DIMENSIONS);
    EXPECT(lev_hip_forge_candidates(ctx, LEV_OP_Q4_0_GEMV, 4096, 8, 2, nullptr, 0, &n) == LEV_ERR_BAD_DIMENSIONS);
    EXPECT(lev_hip_forge_candidates(ctx, LEV_OP_Q4_0_GEMV, 4096, 512, 1, nullptr, 0, &n) == LEV_OK && n == 8);
}

// MoELoweringForge.forge (MoELowering.swift:1896-1985) on the test model's layer 0
void forge_moe_layer(Runner &r, const Model &m) {
    const TensorRef &rt = m.table.at("blk.0.ffn_gate_inp.weight");
    std::vector<float> router((size_t)Model::experts * Model::hidden);
    std::memcpy(router.data(), m.bytes.data() + rt.offset, router.size() * 4);
    for (int tokens : {1, 3}) {
        ForgeOptions opt;
        opt.launchesPerSample = 3;
        opt.timed = 5;
        opt.rotateBytes = 4 << 20;
        ForgeReport rep = MoELayerForge::forge(r, m.bytes, m.binding, router, tokens, opt);
        EXPECT(rep.op == LEV_OP_MOE_LAYER_Q4_0 && rep.candidates.size() == 6);
        EXPECT(rep.candidates[0].schedule.family == 1u && rep.candidates[0].schedule.rows_in_flight == 2u);
        for (const ForgeCandidate &c : rep.candidates) EXPECT(c.pass && c.maxRelErr >= 0 && c.maxRelErr < 1e-4 && c.medianUs > 0);
        EXPECT(rep.selected >= 0 && rep.selected < 6);
        if (rep.selected > 0)
            EXPECT(rep.candidates[(size_t)rep.selected].medianUs < 0.98 * rep.candidates[0].medianUs);
        ForgeOptions strict = opt;
        strict.gate = 0.0;
        EXPECT(MoELayerForge::forge(r, m.bytes, m.binding, router, tokens, strict).selected == -1);
        // leave the built-in choice installed for the cases that follow
        EXPECT(lev_hip_forge_clear(r.context(), LEV_OP_MOE_LAYER_Q4_0, Model::hidden, Model::inter, (uint32_t)tokens) == LEV_OK);
    }
    bool threw = false;
    try {
        MoELayerForge::forge(r, m.bytes, m.binding, router, 5);
    } catch (const Gemma4Error &) {
        threw = true;
    }
    EXPECT(threw);
}

// Gemma4.swift:3742-3773: rmsnorm -> gate, up (one buffer) -> geluUp -> down -> rmsnorm,
// against the same chain on the CPU (FP64 matvecs and norms, f32 between the steps)
void runner_shared_expert(Runner &r, const Model &m) {
    const int H = Model::hidden, I = Model::sharedInter;
    std::vector<float> x(H);
    levo_fill_normal(71, 0.f, 1.f, x.data(), H);
    DeviceBuffer dx = r.makeBuffer(x), dh = r.makeBuffer((int64_t)H * 4), dgu = r.makeBuffer((int64_t)2 * I * 4),
                 dact = r.makeBuffer((int64_t)I * 4), dsh = r.makeBuffer((int64_t)H * 4);
    r.sharedExpert("blk.1.", dx, dh, dgu, dact, dsh, H, I);
    std::vector<float> got = r.read<float>(dsh, H), got_h = r.read<float>(dh, H);

    auto f32 = [](const std::vector<double> &v) { return std::vector<float>(v.begin(), v.end()); };
    auto tensor_bytes = [&](const char *name) { const TensorRef &t = m.table.at(name); return (size_t)(t.end - t.offset); };
    std::vector<double> hd(H), gd(I), ud(I), dd(H), sd(H);
    levo_rmsnorm_f64(x.data(), reinterpret_cast<const float *>(m.at("blk.1.ffn_norm.weight")), 1e-6, H, hd.data());
    EXPECT(rel_err(got_h, hd) < 1e-5);
    std::vector<float> h = f32(hd);
    EXPECT(levo_q4_0_matvec_f64(m.at("blk.1.ffn_gate.weight"), tensor_bytes("blk.1.ffn_gate.weight"), I, H, h.data(), H, gd.data()) == 0);
    EXPECT(levo_q4_0_matvec_f64(m.at("blk.1.ffn_up.weight"), tensor_bytes("blk.1.ffn_up.weight"), I, H, h.data(), H, ud.data()) == 0);
    std::vector<float> g = f32(gd), u = f32(ud), act(I);
    for (int i = 0; i < I; ++i) act[i] = levo_gelu_up_f32(g[i], u[i]);
    EXPECT(levo_q4_0_matvec_f64(m.at("blk.1.ffn_down.weight"), tensor_bytes("blk.1.ffn_down.weight"), H, I, act.data(), I, dd.data()) == 0);
    std::vector<float> d = f32(dd);
    levo_rmsnorm_f64(d.data(), reinterpret_cast<const float *>(m.at("blk.1.post_ffw_norm_1.weight")), 1e-6, H, sd.data());
    EXPECT(rel_err(got, sd) < 1e-4);
    // the two halves of gate|up are where the reference binds them
    std::vector<float> gu = r.read<float>(dgu, (size_t)2 * I);
    EXPECT(rel_err(std::vector<float>(gu.begin(), gu.begin() + I), gd) < 1e-4);
    EXPECT(rel_err(std::vector<float>(gu.begin() + I, gu.end()), ud) < 1e-4);
    // guards: an intermediate size whose up half would not start 256-byte aligned, short buffers
    DeviceBuffer small = r.makeBuffer((int64_t)I * 4);
    EXPECT(throws_geometry([&] { r.sharedExpert("blk.1.", dx, dh, small, dact, dsh, H, I); }));
    EXPECT(throws_geometry([&] { r.sharedExpert("blk.1.", dx, dh, dgu, dact, dsh, H, I - 32); }));
    EXPECT(throws_geometry([&] { r.sharedExpert("blk.7.", dx, dh, dgu, dact, dsh, H, I); }));
    r.flushOpenSegment();
}

int main(int argc, char **argv) {
    Model model;
    std::unique_ptr<Runner> runner;
    auto R = [&]() -> Runner & {
        if (!runner) {
            runner = std::make_unique<Runner>(0);
            runner->bindWeights(model.bytes, model.table);
        }
        return *runner;
    };
    std::vector<Case> cases = {
        {"q4_backend_2x32", q4_backend_2x32},
        {"q4_backend_minus_16", q4_backend_minus_16},
        {"q4_backend_guards", q4_backend_guards},
        {"q6_backend_minus_315", q6_backend_minus_315},
        {"q4_backend_seeded", q4_backend_seeded},
        {"runner_matvec", [&] { runner_matvec(R(), model); }},
        {"runner_elementwise", [&] { runner_elementwise(R(), model); }},
        {"runner_int8_path", [&] { runner_int8_path(R(), model); }},
        {"runner_f32_columns", [&] { runner_f32_columns(R(), model); }},
        {"runner_shared_expert", [&] { runner_shared_expert(R(), model); }},
        {"runner_moe", [&] { runner_moe(R(), model); }},
        {"runner_moe_hand_computed", [&] { runner_moe_hand_computed(R()); }},
        {"runner_gguf_file", [&] { runner_gguf_file(R(), model); }},
        {"forge_matvec", [&] { forge_matvec(R()); }},
        {"forge_moe_layer", [&] { forge_moe_layer(R(), model); }},
    };
    if (argc > 1 && std::strcmp(argv[1], "--list") == 0) {
        for (auto &c : cases) std::printf("%s\n", c.name);
        return 0;
    }
    for (auto &c : cases) {
        std::printf("run %s\n", c.name);
        std::fflush(stdout);
        int before = g_failures;
        try {
            c.run();
        } catch (const std::exception &e) {
            std::printf("FAIL %s: unexpected exception: %s\n", c.name, e.what());
            ++g_failures;
        }
        if (g_failures == before) std::printf("ok %s\n", c.name);
        std::fflush(stdout);
    }
    runner.reset();
    std::printf(g_failures ? "FAILED %d check(s)\n" : "all host parity cases passed\n", g_failures);
    return g_failures ? 1 : 0;
}

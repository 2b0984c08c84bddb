// Host-side mirror, in C++, of the LeviathanCore operator surface that sits
// above the C ABI of libleviathan_hip (include/leviathan_hip.h).
//
// The reference's host side for this path is Swift (Gemma4Runner and the
// standalone Q4MetalBackend / Q6MetalBackend).  This header keeps its names,
// argument meaning and error behaviour so that code and tests written against
// the Swift surface read the same here:
//
//   Q4Error, Q4MatvecEvidence            Sources/LeviathanCore/Q4.swift:17-31, 116-123
//   Q4HipBackend::matvecReporting        Q4MetalBackend.matvecReporting, Q4.swift:165-269
//   Q6HipBackend::matvecReporting        Q6MetalBackend.matvecReporting, Q6.swift:199-285
//   Gemma4Error::badTensorGeometry       Gemma4.swift (thrown by every operator below)
//   Runner::matvec / matvecDispatch      Gemma4.swift:2583, 2638
//   Runner::expertMatvec                 Gemma4.swift:2805 (slice addressing; the slot cache is not mirrored)
//   Runner::rmsnorm / geluUp / axpy      Gemma4.swift:3014, 3103, 3115
//   Runner::normQuant / matvecQ8         Builder::norm_quant / matvec, rust/crates/lev-model/src/gpu.rs:295, 334
//   Runner::embed                        Builder step "embed", gpu.rs:457
//   Runner::bindGGUF / moeBinding        Gemma4.swift:543-566 (resident file), MoEModelBinding.swift:95-214
//   Runner::routeTopK                    Gemma4.swift:3795-3810 (router matvec + softmax/top-k)
//   Runner::runMoeBatchedRouted          Gemma4.swift:2073
//   Runner::flushOpenSegment             Gemma4.swift:2313
//
// Every check the Swift operators make before encoding a command is made here
// before the C ABI is called; the C ABI repeats the extent checks on its own.
// Header-only; link with -lleviathan_hip.
#pragma once

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdint>
#include <cstring>
#include <map>
#include <optional>
#include <set>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "leviathan_gguf.hpp"
#include "leviathan_hip.h"

namespace leviathan {

// ---- Q4.swift:17-31 --------------------------------------------------------
enum class Q4Error : int {
    badDimensions = LEV_ERR_BAD_DIMENSIONS,
    wrongInputCount = LEV_ERR_WRONG_INPUT_COUNT,
    nonFiniteInput = LEV_ERR_NON_FINITE_INPUT,
    nonFiniteScale = LEV_ERR_NON_FINITE_SCALE,
    nonFiniteOutput = LEV_ERR_NON_FINITE_OUTPUT,
    exceedsModelWorkload = LEV_ERR_EXCEEDS_MODEL_WORKLOAD,
    integerOverflow = LEV_ERR_INTEGER_OVERFLOW,
    metalUnavailable = LEV_ERR_DEVICE_UNAVAILABLE,   // "device unavailable" on this backend
    shaderCompileFailed = LEV_ERR_KERNEL_LOAD_FAILED,
    functionMissing = LEV_ERR_FUNCTION_MISSING,
    commandBufferFailed = LEV_ERR_COMMAND_FAILED,
    exceedsMaxBufferLength = LEV_ERR_EXCEEDS_MAX_BUFFER_LENGTH,
    exceedsRecommendedWorkingSet = LEV_ERR_EXCEEDS_WORKING_SET,
    invalidArgument = LEV_ERR_INVALID_ARGUMENT,
};

// Swift `throws Q4Error` becomes a C++ exception carrying the same case.
class Q4Exception : public std::runtime_error {
public:
    Q4Exception(Q4Error c, const std::string &what)
        : std::runtime_error(std::string(lev_hip_status_name((int)c)) + (what.empty() ? "" : ": " + what)),
          code(c) {}
    Q4Error code;
};

// Gemma4Error.badTensorGeometry(String) / .metalUnavailable.
class Gemma4Error : public std::runtime_error {
public:
    enum Kind { badTensorGeometry, metalUnavailable, commandFailed };
    Gemma4Error(Kind k, const std::string &what) : std::runtime_error(what), kind(k) {}
    Kind kind;
};

// ---- Q4.swift:116-123 -------------------------------------------------------
struct Q4MatvecEvidence {
    std::string deviceName;
    uint64_t deviceMaxBufferLength = 0;
    uint64_t recommendedMaxWorkingSetSize = 0;
    int64_t outDim = 0, inDim = 0;
    std::string commandStatus;
};

namespace detail {
inline Q4MatvecEvidence evidence_from(const lev_evidence &e) {
    Q4MatvecEvidence r;
    r.deviceName = e.device_name;
    r.deviceMaxBufferLength = e.device_max_buffer_length;
    r.recommendedMaxWorkingSetSize = e.recommended_max_working_set_size;
    r.outDim = e.out_dim;
    r.inDim = e.in_dim;
    r.commandStatus = e.command_status;
    return r;
}
using reporting_fn = int (*)(const uint8_t *, size_t, int64_t, int64_t, const float *, size_t,
                             float *, lev_evidence *);
inline std::pair<std::vector<float>, Q4MatvecEvidence>
reporting(reporting_fn fn, const std::vector<uint8_t> &blocks, int64_t outDim, int64_t inDim,
          const std::vector<float> &x) {
    std::vector<float> y(outDim > 0 && outDim <= LEV_MAX_Q4_OUTPUT_DIM ? (size_t)outDim : 0);
    lev_evidence ev;
    std::memset(&ev, 0, sizeof ev);
    // non-null pointers even for empty vectors: emptiness is a geometry error, not a null one
    static const uint8_t no_bytes = 0;
    static const float no_floats = 0.f;
    float sink = 0.f;
    int st = fn(blocks.empty() ? &no_bytes : blocks.data(), blocks.size(), outDim, inDim,
                x.empty() ? &no_floats : x.data(), x.size(), y.empty() ? &sink : y.data(), &ev);
    if (st != LEV_OK) throw Q4Exception((Q4Error)st, "");
    return {std::move(y), evidence_from(ev)};
}
}  // namespace detail

// Standalone backends: validate, upload as stored, run, read back, re-check.
struct Q4HipBackend {
    static std::pair<std::vector<float>, Q4MatvecEvidence>
    matvecReporting(const std::vector<uint8_t> &blocks, int64_t outDim, int64_t inDim,
                    const std::vector<float> &x) {
        return detail::reporting(lev_hip_q4_0_matvec_reporting, blocks, outDim, inDim, x);
    }
    static std::vector<float> matvec(const std::vector<uint8_t> &blocks, int64_t outDim, int64_t inDim,
                                     const std::vector<float> &x) {
        return matvecReporting(blocks, outDim, inDim, x).first;
    }
};

struct Q6HipBackend {
    static std::pair<std::vector<float>, Q4MatvecEvidence>
    matvecReporting(const std::vector<uint8_t> &blocks, int64_t outDim, int64_t inDim,
                    const std::vector<float> &x) {
        return detail::reporting(lev_hip_q6_k_matvec_reporting, blocks, outDim, inDim, x);
    }
};

// ---- GGMLTensorType (GGUF.swift:58-91), the subset the runner dispatches ----
enum class GGMLTensorType : int { float32 = LEV_TYPE_F32, float16 = LEV_TYPE_F16, q4_0 = LEV_TYPE_Q4_0,
                                  q4_K = LEV_TYPE_Q4_K, q6_K = LEV_TYPE_Q6_K };

inline int elementsPerBlock(GGMLTensorType t) {
    switch (t) {
    case GGMLTensorType::q4_0: return 32;
    case GGMLTensorType::q4_K:
    case GGMLTensorType::q6_K: return 256;
    default: return 1;
    }
}
inline int bytesPerBlock(GGMLTensorType t) {
    switch (t) {
    case GGMLTensorType::q4_0: return 18;
    case GGMLTensorType::q4_K: return 144;
    case GGMLTensorType::q6_K: return 210;
    case GGMLTensorType::float16: return 2;
    default: return 4;
    }
}

// Gemma4Runner's tensor table entry: where a tensor's bytes sit in the weight
// buffer and its geometry (Gemma4.swift, `ref[tensor]`).
struct TensorRef {
    GGMLTensorType type = GGMLTensorType::q4_0;
    int64_t offset = 0, end = 0;   // byte extent [offset, end) in the weight buffer
    int64_t inDim = 0, outDim = 0;
    int64_t experts = 1;           // 3-D expert tensors: slices of outDim rows each
};

class Runner;

// MTLBuffer analogue: device memory with a byte length the operators check.
class DeviceBuffer {
public:
    DeviceBuffer() = default;
    DeviceBuffer(const DeviceBuffer &) = delete;
    DeviceBuffer &operator=(const DeviceBuffer &) = delete;
    DeviceBuffer(DeviceBuffer &&o) noexcept { *this = std::move(o); }
    DeviceBuffer &operator=(DeviceBuffer &&o) noexcept {
        release();
        ctx_ = o.ctx_; ptr_ = o.ptr_; length = o.length;
        o.ctx_ = nullptr; o.ptr_ = nullptr; o.length = 0;
        return *this;
    }
    ~DeviceBuffer() { release(); }
    void *contents() const { return ptr_; }
    float *floats() const { return static_cast<float *>(ptr_); }
    int64_t length = 0;   // bytes

private:
    friend class Runner;
    void release() {
        if (ptr_ && ctx_) lev_hip_buf_free(ctx_, ptr_);
        ptr_ = nullptr;
    }
    lev_ctx *ctx_ = nullptr;
    void *ptr_ = nullptr;
};

// MoEModelBinding (MoEModelBinding.swift:174-214, 284-292): where the expert
// slices of one layer's gate / up / down tensors sit.
struct MoEBinding {
    int64_t gateOffset = 0, upOffset = 0, downOffset = 0;     // bytes from the weight buffer's start
    int64_t gateStride = 0, upStride = 0, downStride = 0;     // bytes between experts
    int hidden = 0, expertIntermediate = 0, experts = 0, topK = 0;
};

// The operator surface of Gemma4Runner for this path.  One device, one stream
// (the runner's own), deferred execution: operators enqueue, flushOpenSegment()
// waits.  Not thread-safe, as the Swift class.
class Runner {
public:
    explicit Runner(int device = 0, float rmsNormEps = 1e-6f) : eps_(rmsNormEps) {
        int st = lev_hip_ctx_create(device, LEV_HIP_OWN_STREAM, &ctx_);
        if (st != LEV_OK) throw Gemma4Error(Gemma4Error::metalUnavailable, lev_hip_status_name(st));
    }
    Runner(const Runner &) = delete;
    Runner &operator=(const Runner &) = delete;
    ~Runner() {
        weights_ = DeviceBuffer();
        if (ctx_) lev_hip_ctx_destroy(ctx_);
    }

    lev_ctx *context() const { return ctx_; }

    // device.makeBuffer(length:) / makeBuffer(bytes:length:)
    DeviceBuffer makeBuffer(int64_t length) {
        if (length <= 0) throw Gemma4Error(Gemma4Error::badTensorGeometry, "makeBuffer: bad length");
        DeviceBuffer b;
        check(lev_hip_buf_alloc(ctx_, (size_t)length, &b.ptr_), "makeBuffer");
        b.ctx_ = ctx_;
        b.length = length;
        return b;
    }
    template <typename T>
    DeviceBuffer makeBuffer(const std::vector<T> &host) {
        DeviceBuffer b = makeBuffer((int64_t)(host.size() * sizeof(T)));
        check(lev_hip_buf_upload(ctx_, b.ptr_, host.data(), host.size() * sizeof(T)), "upload");
        return b;
    }
    template <typename T>
    std::vector<T> read(const DeviceBuffer &b, size_t count) {
        if ((int64_t)(count * sizeof(T)) > b.length)
            throw Gemma4Error(Gemma4Error::badTensorGeometry, "read beyond buffer");
        flushOpenSegment();
        std::vector<T> out(count);
        check(lev_hip_buf_download(ctx_, out.data(), b.ptr_, count * sizeof(T)), "download");
        return out;
    }

    // Binds the weight bytes exactly as stored (the mapped GGUF data section).
    void bindWeights(const std::vector<uint8_t> &bytes, std::map<std::string, TensorRef> table) {
        weights_ = makeBuffer(bytes);
        mapEnd_ = (int64_t)bytes.size();
        ref_ = std::move(table);
    }

    // Makes a GGUF file resident from offset 0 (buffer offset == file offset, as
    // the reference's mapped file, Gemma4.swift:543-566; uploaded here, since
    // registering mapped host memory is not available) and builds the tensor
    // table from its directory.  Tensors of types this path has no kernel for
    // stay in the buffer but get no table entry.
    GGUFFile bindGGUF(const std::string &path) {
        GGUFFile g = GGUFFile::open(path);
        std::vector<uint8_t> bytes((size_t)g.fileLen);
        FILE *f = std::fopen(path.c_str(), "rb");
        if (!f || std::fread(bytes.data(), 1, bytes.size(), f) != bytes.size()) {
            if (f) std::fclose(f);
            throw GGUFError("cannot read " + path);
        }
        std::fclose(f);
        std::map<std::string, TensorRef> table;
        for (const GGUFTensorInfo &t : g.tensors) {
            TensorRef r;
            switch (t.ggmlType) {
            case LEV_TYPE_F32: r.type = GGMLTensorType::float32; break;
            case LEV_TYPE_F16: r.type = GGMLTensorType::float16; break;
            case LEV_TYPE_Q4_0: r.type = GGMLTensorType::q4_0; break;
            case LEV_TYPE_Q4_K: r.type = GGMLTensorType::q4_K; break;
            case LEV_TYPE_Q6_K: r.type = GGMLTensorType::q6_K; break;
            default: continue;
            }
            uint64_t start, end;
            g.tensorRange(t, start, end);
            r.offset = (int64_t)start;
            r.end = (int64_t)end;
            r.inDim = (int64_t)t.dims[0];
            r.outDim = t.dims.size() > 1 ? (int64_t)t.dims[1] : 1;
            r.experts = t.dims.size() > 2 ? (int64_t)t.dims[2] : 1;
            if (t.dims.size() > 3) continue;
            table[t.name] = r;
        }
        bindWeights(bytes, std::move(table));
        return g;
    }

    // The routed-expert pools of one layer, from the checked file binding
    // (fused gate|up rows [2I, H] per expert: up follows gate inside a slice).
    static MoEBinding moeBinding(const MoEModelBinding &b, int64_t layer) {
        if (layer < 0 || layer >= b.layerCount)
            throw Gemma4Error(Gemma4Error::badTensorGeometry, "layer outside the model");
        MoEBinding m;
        m.gateOffset = b.guTensorStarts[(size_t)layer];
        m.upOffset = m.gateOffset + b.guStride / 2;
        m.downOffset = b.dnTensorStarts[(size_t)layer];
        m.gateStride = m.upStride = b.guStride;
        m.downStride = b.dnStride;
        m.hidden = (int)b.hidden;
        m.expertIntermediate = (int)b.inter;
        m.experts = (int)b.expertCount;
        m.topK = (int)b.topK;
        return m;
    }

    // ---- Gemma4.swift:2583 ----
    void matvec(const std::string &tensor, const DeviceBuffer &x, int64_t xCount, DeviceBuffer &y,
                int64_t yCapacity, int64_t extraOffset = 0, std::optional<int64_t> rows = std::nullopt,
                int64_t yByteOffset = 0) {
        const TensorRef &r = lookup(tensor);
        const int64_t outRows = rows.value_or(r.outDim);
        const int epb = elementsPerBlock(r.type);
        if (!(outRows > 0 && r.inDim > 0 && yByteOffset >= 0 && r.inDim % epb == 0))
            geometry("bad dims for " + tensor);
        int64_t yEnd;
        if (__builtin_add_overflow(yByteOffset, outRows * 4, &yEnd) || yByteOffset % 256 != 0 ||
            y.length < yEnd || yCapacity * 4 < yEnd || x.length < r.inDim * 4)
            geometry("buffer extents violated for " + tensor);
        if (xCount != r.inDim) geometry(tensor + ": input " + std::to_string(xCount) + " != inDim");
        int64_t bytesPerRow, weightBytes, wStart, wEnd;
        if (__builtin_mul_overflow(r.inDim / epb, (int64_t)bytesPerBlock(r.type), &bytesPerRow) ||
            __builtin_mul_overflow(outRows, bytesPerRow, &weightBytes) ||
            __builtin_add_overflow(r.offset, extraOffset, &wStart) ||
            __builtin_add_overflow(wStart, weightBytes, &wEnd) || wStart < r.offset || wEnd > r.end ||
            wEnd > mapEnd_)
            geometry(tensor + ": weight bytes beyond tensor extent");
        if (!weights_.contents()) throw Gemma4Error(Gemma4Error::metalUnavailable, "no weights bound");
        matvecDispatch(tensor, r.type, weights_, wStart, r.inDim, outRows, x, y, yByteOffset);
    }

    // ---- Gemma4.swift:2638: kernel selection; extents are the caller's job ----
    void matvecDispatch(const std::string &tensor, GGMLTensorType type, const DeviceBuffer &wbase,
                        int64_t wStart, int64_t inDim, int64_t outRows, const DeviceBuffer &x,
                        DeviceBuffer &y, int64_t yByteOffset) {
        float *yp = reinterpret_cast<float *>(static_cast<char *>(y.contents()) + yByteOffset);
        const size_t ycap = (size_t)((y.length - yByteOffset) / 4);
        switch (type) {
        case GGMLTensorType::q4_0:
            check(lev_hip_q4_0_gemv(ctx_, wbase.contents(), (size_t)wbase.length, (uint64_t)wStart,
                                    x.floats(), (size_t)inDim, yp, ycap, (uint32_t)inDim,
                                    (uint32_t)outRows), tensor);
            return;
        case GGMLTensorType::q6_K:
            check(lev_hip_q6_k_gemv(ctx_, wbase.contents(), (size_t)wbase.length, (uint64_t)wStart,
                                    x.floats(), (size_t)inDim, yp, ycap, (uint32_t)inDim,
                                    (uint32_t)outRows, nullptr, nullptr), tensor);
            return;
        case GGMLTensorType::q4_K:
            check(lev_hip_q4_k_gemv_ncol(ctx_, wbase.contents(), (size_t)wbase.length, (uint64_t)wStart,
                                         x.floats(), (size_t)inDim, nullptr, 0.f, yp, ycap,
                                         (uint32_t)inDim, (uint32_t)outRows, 1), tensor);
            return;
        case GGMLTensorType::float16:
            geometry("F16 unsupported for " + tensor);
        default:
            geometry("no kernel for the type of " + tensor);
        }
    }

    // ---- Gemma4.swift:2805: one expert's slice of a 3-D Q4_0 tensor ----
    void expertMatvec(const std::string &tensor, int64_t layer, int64_t expert, const DeviceBuffer &x,
                      int64_t xCount, DeviceBuffer &y, int64_t yCapacity) {
        const std::string gu = "blk." + std::to_string(layer) + ".ffn_gate_up_exps.weight";
        const std::string dn = "blk." + std::to_string(layer) + ".ffn_down_exps.weight";
        if (tensor != gu && tensor != dn)
            geometry("expertMatvec requires blk.<layer>.ffn_{gate_up,down}_exps.weight, got " + tensor);
        auto it = ref_.find(tensor);
        if (it == ref_.end() || it->second.type != GGMLTensorType::q4_0)
            geometry("missing/mistyped expert tensor " + tensor);
        const TensorRef &r = it->second;
        if (!(expert >= 0 && expert < r.experts && layer >= 0))
            geometry(tensor + ": expert " + std::to_string(expert) + " out of bounds");
        int64_t bytesPerRow, stride, prod, wStart, wEnd;
        if (__builtin_mul_overflow(r.inDim / 32, (int64_t)18, &bytesPerRow) ||
            __builtin_mul_overflow(r.outDim, bytesPerRow, &stride) || stride <= 0 ||
            xCount != r.inDim || x.length < r.inDim * 4 || y.length < r.outDim * 4 ||
            yCapacity < r.outDim)
            geometry(tensor + ": slice/buffer geometry mismatch");
        if (__builtin_mul_overflow(expert, stride, &prod) ||
            __builtin_add_overflow(r.offset, prod, &wStart) ||
            __builtin_add_overflow(wStart, stride, &wEnd) || wStart < r.offset || wEnd > r.end)
            geometry(tensor + ": slice beyond tensor extent");
        matvecDispatch(tensor, r.type, weights_, wStart, r.inDim, r.outDim, x, y, 0);
    }

    // ---- Gemma4.swift:3014 ----
    void rmsnorm(const DeviceBuffer &x, DeviceBuffer &y, int64_t n, int64_t vectors,
                 const std::optional<std::string> &weightTensor) {
        const float *w = nullptr;
        if (weightTensor) {
            auto it = ref_.find(*weightTensor);
            if (it == ref_.end() || it->second.type != GGMLTensorType::float32 ||
                it->second.inDim != n || it->second.end - it->second.offset != n * 4)
                geometry("bad norm weight " + *weightTensor);
            w = reinterpret_cast<const float *>(static_cast<const char *>(weights_.contents()) +
                                                it->second.offset);
        }
        int64_t span;
        if (__builtin_mul_overflow(n, vectors * 4, &span) || n <= 0 || vectors <= 0 ||
            x.length < span || y.length < span)
            geometry("rmsnorm buffers too small");
        check(lev_hip_rmsnorm(ctx_, x.floats(), y.floats(), (uint32_t)n, (uint32_t)vectors, w, eps_),
              "rmsnorm");
    }

    // ---- Builder step "embed", rust/crates/lev-model/src/gpu.rs:457 (embed_q4k, lev-forge/src/ops.rs:523) ----
    // out[nb][dim] = rows tokens[0..nb) of a Q4_K table [vocab][dim]; tokens are u32 on the device.
    void embed(const std::string &tensor, const DeviceBuffer &tokens, int64_t nb, DeviceBuffer &out) {
        const TensorRef &r = lookup(tensor);
        int64_t count;
        if (r.type != GGMLTensorType::q4_K || r.inDim <= 0 || r.inDim % 256 != 0 || r.outDim <= 0 || nb <= 0 ||
            __builtin_mul_overflow(r.inDim, nb, &count) || tokens.length < nb * 4 || out.length < count * 4)
            geometry("embed: " + tensor + " is not a Q4_K table or the buffers are too small");
        check(lev_hip_embed_q4_k(ctx_, weights_.contents(), (size_t)weights_.length, (uint64_t)r.offset,
                                 static_cast<const uint32_t *>(tokens.contents()), (uint32_t)nb, out.floats(),
                                 (size_t)(out.length / 4), (uint32_t)r.inDim, (uint32_t)r.outDim),
              tensor);
    }

    // ---- Builder::norm_quant, rust/crates/lev-model/src/gpu.rs:295-320 ----
    // x [nb][ne] += add (if given, written back), RMS norm with the weight
    // tensor (if given; otherwise the plain quantiser, gpu.rs:282-290), int8
    // codes into xq [nb][ne], (d, s) pairs into xs [nb][ne/32]; y (if given)
    // also receives the f32 result.
    void normQuant(DeviceBuffer &x, int64_t ne, int64_t nb, const std::optional<std::string> &weightTensor,
                   DeviceBuffer &xq, DeviceBuffer &xs, const DeviceBuffer *add = nullptr,
                   DeviceBuffer *y = nullptr) {
        const float *w = nullptr;
        if (weightTensor) {
            auto it = ref_.find(*weightTensor);
            if (it == ref_.end() || it->second.type != GGMLTensorType::float32 ||
                it->second.inDim != ne || it->second.end - it->second.offset != ne * 4)
                geometry("bad norm weight " + *weightTensor);
            w = reinterpret_cast<const float *>(static_cast<const char *>(weights_.contents()) +
                                                it->second.offset);
        }
        int64_t count;
        if (ne <= 0 || nb <= 0 || ne % 32 != 0 || __builtin_mul_overflow(ne, nb, &count) ||
            x.length < count * 4 || xq.length < count || xs.length < count / 32 * 8 ||
            (add && add->length < count * 4) || (y && y->length < count * 4))
            geometry("norm_quant buffers too small");
        check(lev_hip_norm_quant_q8(ctx_, x.floats(), (size_t)count, add ? add->floats() : nullptr, w, eps_,
                                    static_cast<int8_t *>(xq.contents()), xs.floats(),
                                    y ? y->floats() : nullptr, (uint32_t)ne, (uint32_t)nb),
              "norm_quant");
    }

    // ---- Builder::matvec / matvec_rows on int8 activations, gpu.rs:334-370 ----
    // y[nb][rows] (from float index yOffset) = W x for a Q4_K or Q6_K tensor; reads the
    // activations quantised by normQuant; maxRows takes a prefix of the rows.
    void matvecQ8(const std::string &tensor, const DeviceBuffer &xq, const DeviceBuffer &xs, int64_t nb,
                  DeviceBuffer &y, int64_t yOffset = 0, std::optional<int64_t> maxRows = std::nullopt) {
        const TensorRef &r = lookup(tensor);
        if (r.type != GGMLTensorType::q4_K && r.type != GGMLTensorType::q6_K)
            geometry(tensor + ": unsupported type for the int8 matvec");
        const int64_t blockBytes = bytesPerBlock(r.type);
        const int64_t rows = std::min(r.outDim, maxRows.value_or(r.outDim));
        int64_t count, outs, weightBytes, wEnd;
        if (!(rows > 0 && r.inDim > 0 && r.inDim % 256 == 0 && nb > 0 && yOffset >= 0) ||
            __builtin_mul_overflow(r.inDim, nb, &count) || __builtin_mul_overflow(rows, nb, &outs) ||
            xq.length < count || xs.length < count / 32 * 8 || y.length < (yOffset + outs) * 4)
            geometry("buffer extents violated for " + tensor);
        if (__builtin_mul_overflow(rows, r.inDim / 256 * blockBytes, &weightBytes) ||
            __builtin_add_overflow(r.offset, weightBytes, &wEnd) || wEnd > r.end || wEnd > mapEnd_)
            geometry(tensor + ": weight bytes beyond tensor extent");
        auto *kernel = r.type == GGMLTensorType::q4_K ? lev_hip_q4_k_gemv_q8 : lev_hip_q6_k_gemv_q8;
        check(kernel(ctx_, weights_.contents(), (size_t)weights_.length, (uint64_t)r.offset,
                     static_cast<const int8_t *>(xq.contents()), xs.floats(), (size_t)count,
                     y.floats() + yOffset, (size_t)(y.length / 4 - yOffset), (uint32_t)r.inDim, (uint32_t)rows,
                     (uint32_t)nb),
              tensor);
    }

    // ---- Builder::norm_quant + Builder::matvec on f32 activations, gpu.rs:295, 334-370 ----
    // y[nb][rows] (from float index yOffset) = W rmsnorm(x[nb][inDim]) * gain for a Q4_K or
    // Q6_K tensor, every column per one pass over the weights; no gain tensor: y = W x.
    // Sums are formed without rounding, so a column does not depend on its companions.
    void matvecCols(const std::string &tensor, const DeviceBuffer &x, int64_t nb, DeviceBuffer &y,
                    const std::optional<std::string> &gainTensor = std::nullopt, int64_t yOffset = 0,
                    std::optional<int64_t> maxRows = std::nullopt) {
        const TensorRef &r = lookup(tensor);
        if (r.type != GGMLTensorType::q4_K && r.type != GGMLTensorType::q6_K)
            geometry(tensor + ": unsupported type for the multi-column matvec");
        const float *g = nullptr;
        if (gainTensor) {
            auto it = ref_.find(*gainTensor);
            if (it == ref_.end() || it->second.type != GGMLTensorType::float32 ||
                it->second.inDim != r.inDim || it->second.end - it->second.offset != r.inDim * 4)
                geometry("bad norm weight " + *gainTensor);
            g = reinterpret_cast<const float *>(static_cast<const char *>(weights_.contents()) +
                                                it->second.offset);
        }
        const int64_t blockBytes = bytesPerBlock(r.type);
        const int64_t rows = std::min(r.outDim, maxRows.value_or(r.outDim));
        int64_t count, outs, weightBytes, wEnd;
        if (!(rows > 0 && r.inDim > 0 && r.inDim % 256 == 0 && nb > 0 && yOffset >= 0) ||
            __builtin_mul_overflow(r.inDim, nb, &count) || __builtin_mul_overflow(rows, nb, &outs) ||
            x.length < count * 4 || y.length < (yOffset + outs) * 4)
            geometry("buffer extents violated for " + tensor);
        if (__builtin_mul_overflow(rows, r.inDim / 256 * blockBytes, &weightBytes) ||
            __builtin_add_overflow(r.offset, weightBytes, &wEnd) || wEnd > r.end || wEnd > mapEnd_)
            geometry(tensor + ": weight bytes beyond tensor extent");
        auto *kernel = r.type == GGMLTensorType::q4_K ? lev_hip_q4_k_gemv_ncol : lev_hip_q6_k_gemv_ncol;
        check(kernel(ctx_, weights_.contents(), (size_t)weights_.length, (uint64_t)r.offset, x.floats(),
                     (size_t)count, g, eps_, y.floats() + yOffset, (size_t)(y.length / 4 - yOffset),
                     (uint32_t)r.inDim, (uint32_t)rows, (uint32_t)nb),
              tensor);
    }

    // ---- Gemma4.swift:3103 ----
    void geluUp(const DeviceBuffer &gu, DeviceBuffer &y, int64_t n) {
        if (n <= 0 || gu.length < 2 * n * 4 || y.length < n * 4)
            geometry("gelu_up buffer too small for n=" + std::to_string(n));
        check(lev_hip_gelu_up(ctx_, gu.floats(), y.floats(), (uint32_t)n), "gelu_up");
    }

    // ---- Gemma4.swift:3115 ----
    void axpy(const DeviceBuffer &x, DeviceBuffer &y, float c, int64_t n, int64_t xOffset = 0) {
        if (!(n > 0 && n <= (int64_t)UINT32_MAX && xOffset >= 0 && xOffset % 4 == 0 && std::isfinite(c)))
            geometry("axpy bounds: n=" + std::to_string(n) + " xOffset=" + std::to_string(xOffset));
        int64_t n4, span;
        if (__builtin_mul_overflow(n, (int64_t)4, &n4) || __builtin_add_overflow(n4, xOffset, &span) ||
            x.length < span || y.length < n4)
            geometry("axpy buffer too small");
        const float *xp = reinterpret_cast<const float *>(static_cast<const char *>(x.contents()) + xOffset);
        check(lev_hip_axpy(ctx_, xp, y.floats(), c, (uint32_t)n), "axpy");
    }

    // ---- Gemma4.swift:3742-3773: the shared expert beside the routed ones ----
    // bufH = rmsnorm(bufX, ffn_norm); gate|up fused into bufGU ([0..I) gate, [I..2I) up through a
    // 256-aligned byte offset); bufAct = geluUp(bufGU); bufShared = rmsnorm(down bufAct,
    // post_ffw_norm_1).  bufH is left holding the normed input for the routed experts.
    void sharedExpert(const std::string &prefix, const DeviceBuffer &bufX, DeviceBuffer &bufH,
                      DeviceBuffer &bufGU, DeviceBuffer &bufAct, DeviceBuffer &bufShared, int64_t hidden,
                      int64_t sharedIntermediate) {
        rmsnorm(bufX, bufH, hidden, 1, prefix + "ffn_norm.weight");
        matvec(prefix + "ffn_gate.weight", bufH, hidden, bufGU, 2 * sharedIntermediate);
        matvec(prefix + "ffn_up.weight", bufH, hidden, bufGU, 2 * sharedIntermediate, 0, std::nullopt,
               sharedIntermediate * 4);
        geluUp(bufGU, bufAct, sharedIntermediate);
        matvec(prefix + "ffn_down.weight", bufAct, sharedIntermediate, bufShared, hidden);
        rmsnorm(bufShared, bufShared, hidden, 1, prefix + "post_ffw_norm_1.weight");
    }

    // ---- Gemma4.swift:3795-3810: router scores, softmax, top-k, renormalise ----
    // routerTensor is F32 [experts][hidden].  Returns (topIdx, weights) for one token.
    std::pair<std::vector<int>, std::vector<float>>
    routeTopK(const std::string &routerTensor, const DeviceBuffer &x, int topK) {
        const TensorRef &r = lookup(routerTensor);
        if (r.type != GGMLTensorType::float32 || r.inDim <= 0 || r.outDim <= 0 ||
            r.end - r.offset != r.inDim * r.outDim * 4 || x.length < r.inDim * 4 || topK <= 0 ||
            topK > r.outDim)
            geometry("bad router tensor " + routerTensor);
        DeviceBuffer ids = makeBuffer((int64_t)topK * 4), wts = makeBuffer((int64_t)topK * 4);
        const float *wr = reinterpret_cast<const float *>(static_cast<const char *>(weights_.contents()) +
                                                          r.offset);
        check(lev_hip_moe_route_topk(ctx_, wr, x.floats(), nullptr, static_cast<int32_t *>(ids.contents()),
                                     wts.floats(), nullptr, (uint32_t)r.inDim, (uint32_t)r.outDim,
                                     (uint32_t)topK, 1), "router");
        std::vector<int32_t> hi = read<int32_t>(ids, (size_t)topK);
        std::vector<float> hw = read<float>(wts, (size_t)topK);
        return {std::vector<int>(hi.begin(), hi.end()), hw};
    }

    // ---- Gemma4.swift:2073 ----
    // y = sum over slots, in slot order, of weights[k] * down_e(gelu(gate_e x) * up_e x).
    void runMoeBatchedRouted(const DeviceBuffer &x, DeviceBuffer &y, const std::vector<int> &topIdx,
                             const std::vector<float> &weights, const MoEBinding &binding) {
        if (binding.topK <= 0 || binding.hidden <= 0 || binding.expertIntermediate <= 0 ||
            binding.experts <= 0)
            geometry("installed MoE region dims disagree with this model");
        if (x.length < (int64_t)binding.hidden * 4 || y.length < (int64_t)binding.hidden * 4)
            geometry("batched routed buffers too small for hidden " + std::to_string(binding.hidden));
        if (x.contents() == y.contents()) geometry("routed input aliases the accumulator");
        if ((int)weights.size() != binding.topK)
            geometry("routed merge weights must be " + std::to_string(binding.topK) + " finite values");
        for (float w : weights)
            if (!std::isfinite(w))
                geometry("routed merge weights must be " + std::to_string(binding.topK) + " finite values");
        // MoEModelBinding.offsets: exactly topK ids, in range, distinct
        if ((int)topIdx.size() != binding.topK) geometry("expert id count != topK");
        std::set<int> seen;
        for (int e : topIdx) {
            if (e < 0 || e >= binding.experts) geometry("expert id out of range");
            if (!seen.insert(e).second) geometry("duplicate expert id");
        }
        lev_moe_experts pools;
        pools.d_base = weights_.contents();
        pools.base_bytes = (size_t)weights_.length;
        pools.gate_off = (uint64_t)binding.gateOffset;
        pools.up_off = (uint64_t)binding.upOffset;
        pools.down_off = (uint64_t)binding.downOffset;
        pools.gate_stride = (uint64_t)binding.gateStride;
        pools.up_stride = (uint64_t)binding.upStride;
        pools.down_stride = (uint64_t)binding.downStride;
        pools.hidden = (uint32_t)binding.hidden;
        pools.inter = (uint32_t)binding.expertIntermediate;
        pools.experts = (uint32_t)binding.experts;
        std::vector<int32_t> ids32(topIdx.begin(), topIdx.end());
        // the route buffers must outlive the enqueued kernels: keep them until the next flush
        route_bufs_.push_back(makeBuffer(ids32));
        route_bufs_.push_back(makeBuffer(weights));
        const DeviceBuffer &dIds = route_bufs_[route_bufs_.size() - 2];
        const DeviceBuffer &dW = route_bufs_[route_bufs_.size() - 1];
        check(lev_hip_moe_experts_q4_0(ctx_, &pools, x.floats(), static_cast<const int32_t *>(dIds.contents()),
                                       dW.floats(), y.floats(), nullptr, (uint32_t)binding.topK, 1),
              "runMoeBatchedRouted");
    }

    // ---- Gemma4.swift:2313: commit the deferred segment and wait ----
    void flushOpenSegment() {
        int st = lev_hip_sync(ctx_);
        route_bufs_.clear();
        if (st != LEV_OK)
            throw Gemma4Error(st == LEV_ERR_BAD_DIMENSIONS ? Gemma4Error::badTensorGeometry
                                                           : Gemma4Error::commandFailed,
                              lev_hip_last_error(ctx_));
    }

private:
    [[noreturn]] static void geometry(const std::string &what) {
        throw Gemma4Error(Gemma4Error::badTensorGeometry, what);
    }
    const TensorRef &lookup(const std::string &tensor) const {
        auto it = ref_.find(tensor);
        if (it == ref_.end()) geometry("missing " + tensor);
        return it->second;
    }
    void check(int st, const std::string &what) {
        if (st == LEV_OK) return;
        const std::string msg = what + ": " + lev_hip_last_error(ctx_);
        switch (st) {
        case LEV_ERR_DEVICE_UNAVAILABLE: throw Gemma4Error(Gemma4Error::metalUnavailable, msg);
        case LEV_ERR_COMMAND_FAILED: throw Gemma4Error(Gemma4Error::commandFailed, msg);
        default: throw Gemma4Error(Gemma4Error::badTensorGeometry, msg);
        }
    }

    lev_ctx *ctx_ = nullptr;
    float eps_;
    DeviceBuffer weights_;
    int64_t mapEnd_ = 0;
    std::map<std::string, TensorRef> ref_;
    std::vector<DeviceBuffer> route_bufs_;
};

}  // namespace leviathan

// Host-array twins of the reference's standalone backends:
//   Q4MetalBackend.matvecReporting   Sources/LeviathanCore/Q4.swift:165-269
//   Q6MetalBackend.matvecReporting   Sources/LeviathanCore/Q6.swift:199-285
// Same order of checks, same failure cases, everything validated before any
// device call; the weights are uploaded exactly as stored.
#include "lev_common.hpp"

#include <cmath>

hipError_t lev_q4_0_gemv_launch(lev_ctx *ctx, const uint8_t *w, const float *x, float *y,
                                uint32_t in_dim, uint32_t rows);
hipError_t lev_q6_k_gemv_launch(lev_ctx *ctx, const uint8_t *w, const float *x, float *y,
                                uint32_t in_dim, uint32_t rows);

namespace {

struct device_buffers {
    lev_ctx *ctx = nullptr;
    void *w = nullptr, *x = nullptr, *y = nullptr;
    ~device_buffers() {
        if (ctx) {
            lev_hip_buf_free(ctx, w);
            lev_hip_buf_free(ctx, x);
            lev_hip_buf_free(ctx, y);
            lev_hip_ctx_destroy(ctx);
        }
    }
};

int matvec_reporting(bool q6, const uint8_t *blocks, size_t blocks_count, int64_t out_dim,
                     int64_t in_dim, const float *x, size_t x_count, float *y_out,
                     lev_evidence *evidence) {
    const int64_t values = q6 ? 256 : 32, bytes = q6 ? 210 : 18;
    // geometry (Q4.swift:168-172)
    if (in_dim <= 0 || out_dim <= 0 || in_dim % values != 0 || in_dim > LEV_MAX_Q4_INPUT_DIM ||
        out_dim > LEV_MAX_Q4_OUTPUT_DIM)
        return LEV_ERR_BAD_DIMENSIONS;
    // kernel parameters are 32-bit (Q4.swift:173-175); implied by the caps above
    if (in_dim > (int64_t)UINT32_MAX || out_dim > (int64_t)UINT32_MAX) return LEV_ERR_INTEGER_OVERFLOW;
    // weight byte count (Q4.swift:176-185)
    int64_t row_bytes, weight_bytes;
    if (__builtin_mul_overflow(in_dim / values, bytes, &row_bytes) ||
        __builtin_mul_overflow(out_dim, row_bytes, &weight_bytes) ||
        (uint64_t)weight_bytes > LEV_MAX_Q4_WEIGHT_BYTES || (int64_t)blocks_count != weight_bytes)
        return LEV_ERR_BAD_DIMENSIONS;
    if ((int64_t)x_count != in_dim) return LEV_ERR_WRONG_INPUT_COUNT;
    if (!blocks || !x || !y_out) return LEV_ERR_INVALID_ARGUMENT;
    for (int64_t i = 0; i < in_dim; ++i)
        if (!std::isfinite(x[i])) return LEV_ERR_NON_FINITE_INPUT;

    device_buffers b;
    int st = lev_hip_ctx_create(0, LEV_HIP_OWN_STREAM, &b.ctx);
    if (st != LEV_OK) return st;
    // device limits before any allocation (Q4.swift:197-209)
    size_t free_b = 0, total_b = 0;
    if (hipMemGetInfo(&free_b, &total_b) != hipSuccess) return LEV_ERR_DEVICE_UNAVAILABLE;
    if ((uint64_t)weight_bytes > total_b) return LEV_ERR_EXCEEDS_MAX_BUFFER_LENGTH;
    int64_t total_needed;
    if (__builtin_add_overflow(weight_bytes, in_dim * 4 + out_dim * 4, &total_needed) ||
        (uint64_t)total_needed > free_b)
        return LEV_ERR_EXCEEDS_WORKING_SET;

    if ((st = lev_hip_buf_alloc(b.ctx, (size_t)weight_bytes, &b.w)) != LEV_OK) return st;
    if ((st = lev_hip_buf_alloc(b.ctx, (size_t)in_dim * 4, &b.x)) != LEV_OK) return st;
    if ((st = lev_hip_buf_alloc(b.ctx, (size_t)out_dim * 4, &b.y)) != LEV_OK) return st;
    if ((st = lev_hip_buf_upload(b.ctx, b.w, blocks, (size_t)weight_bytes)) != LEV_OK) return st;
    if ((st = lev_hip_buf_upload(b.ctx, b.x, x, (size_t)in_dim * 4)) != LEV_OK) return st;
    hipError_t e = q6 ? lev_q6_k_gemv_launch(b.ctx, static_cast<const uint8_t *>(b.w),
                                             static_cast<const float *>(b.x),
                                             static_cast<float *>(b.y), (uint32_t)in_dim,
                                             (uint32_t)out_dim)
                      : lev_q4_0_gemv_launch(b.ctx, static_cast<const uint8_t *>(b.w),
                                             static_cast<const float *>(b.x),
                                             static_cast<float *>(b.y), (uint32_t)in_dim,
                                             (uint32_t)out_dim);
    if (e != hipSuccess) return LEV_ERR_COMMAND_FAILED;
    if ((st = lev_hip_sync(b.ctx)) != LEV_OK) return LEV_ERR_COMMAND_FAILED;
    if ((st = lev_hip_buf_download(b.ctx, y_out, b.y, (size_t)out_dim * 4)) != LEV_OK) return st;
    for (int64_t i = 0; i < out_dim; ++i)
        if (!std::isfinite(y_out[i])) return LEV_ERR_NON_FINITE_OUTPUT;
    if (evidence) {
        std::memset(evidence, 0, sizeof(*evidence));
        std::snprintf(evidence->device_name, sizeof(evidence->device_name), "%s (%s)",
                      b.ctx->props.name, b.ctx->props.gcnArchName);
        evidence->device_max_buffer_length = total_b;
        evidence->recommended_max_working_set_size = free_b;
        evidence->out_dim = out_dim;
        evidence->in_dim = in_dim;
        std::snprintf(evidence->command_status, sizeof(evidence->command_status), "completed");
    }
    return LEV_OK;
}

}  // namespace

extern "C" int lev_hip_q4_0_matvec_reporting(const uint8_t *blocks, size_t blocks_count,
                                             int64_t out_dim, int64_t in_dim, const float *x,
                                             size_t x_count, float *y_out, lev_evidence *evidence) {
    return matvec_reporting(false, blocks, blocks_count, out_dim, in_dim, x, x_count, y_out, evidence);
}

extern "C" int lev_hip_q6_k_matvec_reporting(const uint8_t *blocks, size_t blocks_count,
                                             int64_t out_dim, int64_t in_dim, const float *x,
                                             size_t x_count, float *y_out, lev_evidence *evidence) {
    return matvec_reporting(true, blocks, blocks_count, out_dim, in_dim, x, x_count, y_out, evidence);
}

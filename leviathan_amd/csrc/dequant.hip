// Block dequantisation to f32, bit-exact with the reference decoders:
//   Q4_0  Q4_0.decodeBlock            Sources/LeviathanCore/Q4.swift:54-69
//   Q6_K  Q6_K.decodeBlock            Sources/LeviathanCore/Q6.swift:23-62
//   Q4_K  dequant_block_f32           rust/crates/lev-cpu/src/lib.rs:111-131
// One thread per output value; the arithmetic keeps the reference's order of
// operations and is compiled without fused multiply-add.
#include "lev_common.hpp"

#pragma clang fp contract(off)

namespace {

__global__ void __launch_bounds__(256)
dequant_q4_0(const uint8_t *__restrict__ w, float *__restrict__ out, uint64_t nvalues) {
    uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= nvalues) return;
    const uint8_t *blk = w + (i >> 5) * 18u;
    uint32_t e = (uint32_t)(i & 31u);
    float d = lev_f16_bits_to_f32((uint32_t)blk[0] | ((uint32_t)blk[1] << 8));
    uint8_t byte = blk[2 + (e & 15u)];
    float n = (float)(e < 16 ? (byte & 0xF) : (byte >> 4));
    out[i] = d * (n - 8.0f);
}

__global__ void __launch_bounds__(256)
dequant_q6_k(const uint8_t *__restrict__ w, float *__restrict__ out, uint64_t nvalues) {
    uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= nvalues) return;
    const uint8_t *blk = w + (i >> 8) * 210u;
    uint32_t e = (uint32_t)(i & 255u);
    uint32_t half = e >> 7, r = e & 127u, grp = r >> 5, l = r & 31u;
    float d = lev_f16_bits_to_f32((uint32_t)blk[208] | ((uint32_t)blk[209] << 8));
    uint8_t ql = blk[half * 64 + (grp & 1u) * 32 + l];
    uint32_t low = grp < 2 ? (ql & 0xFu) : (ql >> 4);
    uint32_t two = (blk[128 + half * 32 + l] >> (2 * grp)) & 3u;
    int level = (int)(low | (two << 4)) - 32;
    float sc = (float)(int)(int8_t)blk[192 + (e >> 4)];
    out[i] = d * sc * (float)level;
}

__device__ __forceinline__ void q4_k_scale_min(uint32_t j, const uint8_t *s, uint32_t &sc,
                                               uint32_t &mn) {
    if (j < 4) {
        sc = s[j] & 63u;
        mn = s[j + 4] & 63u;
    } else {
        sc = (s[j + 4] & 0x0Fu) | ((uint32_t)(s[j - 4] >> 6) << 4);
        mn = (uint32_t)(s[j + 4] >> 4) | ((uint32_t)(s[j] >> 6) << 4);
    }
}

__global__ void __launch_bounds__(256)
dequant_q4_k(const uint8_t *__restrict__ w, float *__restrict__ out, uint64_t nvalues) {
    uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= nvalues) return;
    const uint8_t *blk = w + (i >> 8) * 144u;
    uint32_t e = (uint32_t)(i & 255u);
    uint32_t j = e >> 5, l = e & 31u;
    float d = lev_f16_bits_to_f32((uint32_t)blk[0] | ((uint32_t)blk[1] << 8));
    float dmin = lev_f16_bits_to_f32((uint32_t)blk[2] | ((uint32_t)blk[3] << 8));
    uint32_t sc, mn;
    q4_k_scale_min(j, blk + 4, sc, mn);
    uint8_t q = blk[16 + (j >> 1) * 32 + l];
    float n = (float)((j & 1u) ? (q >> 4) : (q & 0xF));
    float d1 = d * (float)sc;
    float mm = dmin * (float)mn;
    out[i] = d1 * n - mm;
}

// Embedding lookup from a Q4_K table (embed_q4k, lev-forge/src/ops.rs:523-555):
// column c of out is row tok[c], one workgroup per 256-weight block, the
// arithmetic of dequant_q4_k above.  A token id beyond the table raises the
// context's flag (bit 2) and writes nothing.
constexpr int kFlagBadToken = 4;

__global__ void __launch_bounds__(256)
embed_q4_k(const uint8_t *__restrict__ w, const uint32_t *__restrict__ tok, float *__restrict__ out,
           uint32_t blocks_per_row, uint32_t vocab, int *__restrict__ flag) {
    const uint32_t col = blockIdx.x / blocks_per_row, b = blockIdx.x - col * blocks_per_row;
    const uint32_t token = tok[col];
    if (token >= vocab) {
        if (threadIdx.x == 0 && b == 0) atomicOr(flag, kFlagBadToken);
        return;
    }
    const uint8_t *blk = w + ((uint64_t)token * blocks_per_row + b) * 144u;
    const uint32_t e = threadIdx.x, j = e >> 5, l = e & 31u;
    float d = lev_f16_bits_to_f32((uint32_t)blk[0] | ((uint32_t)blk[1] << 8));
    float dmin = lev_f16_bits_to_f32((uint32_t)blk[2] | ((uint32_t)blk[3] << 8));
    uint32_t sc, mn;
    q4_k_scale_min(j, blk + 4, sc, mn);
    uint8_t q = blk[16 + (j >> 1) * 32 + l];
    float n = (float)((j & 1u) ? (q >> 4) : (q & 0xF));
    float d1 = d * (float)sc;
    float mm = dmin * (float)mn;
    out[((uint64_t)col * blocks_per_row + b) * 256u + e] = d1 * n - mm;
}

}  // namespace

extern "C" int lev_hip_embed_q4_k(lev_ctx *ctx, const void *d_w, size_t w_bytes, uint64_t w_off,
                                  const uint32_t *d_tokens, uint32_t ntokens, float *d_out,
                                  size_t out_capacity, uint32_t dim, uint32_t vocab) {
    LEV_REQUIRE_CTX(ctx);
    if (!d_w || !d_tokens || !d_out) return lev_fail(ctx, LEV_ERR_INVALID_ARGUMENT, "embed_q4_k: null pointer");
    if (dim == 0 || dim % 256u != 0u || dim > LEV_MAX_Q4_INPUT_DIM || vocab == 0 || ntokens == 0 ||
        ntokens > (1u << 20))
        return lev_fail(ctx, LEV_ERR_BAD_DIMENSIONS, "embed_q4_k: dim %u (multiple of 256), vocab %u, %u tokens",
                        dim, vocab, ntokens);
    uint64_t need, end;
    if (__builtin_mul_overflow((uint64_t)vocab, (uint64_t)(dim / 256u) * 144u, &need) ||
        __builtin_add_overflow(w_off, need, &end))
        return lev_fail(ctx, LEV_ERR_INTEGER_OVERFLOW, "embed_q4_k: extent overflows");
    if (end > w_bytes || need > LEV_MAX_Q4_WEIGHT_BYTES)
        return lev_fail(ctx, LEV_ERR_BAD_DIMENSIONS, "embed_q4_k: table [%llu, %llu) beyond %zu bytes",
                        (unsigned long long)w_off, (unsigned long long)end, w_bytes);
    if (out_capacity < (uint64_t)ntokens * dim)
        return lev_fail(ctx, LEV_ERR_BAD_DIMENSIONS, "embed_q4_k: out holds %zu, needs %llu", out_capacity,
                        (unsigned long long)ntokens * dim);
    const uint64_t groups = (uint64_t)ntokens * (dim / 256u);
    if (groups > 0x7FFFFFFFull) return lev_fail(ctx, LEV_ERR_EXCEEDS_MODEL_WORKLOAD, "embed_q4_k: grid");
    hipLaunchKernelGGL(embed_q4_k, dim3((unsigned)groups), dim3(256), 0, ctx->stream,
                       static_cast<const uint8_t *>(d_w) + w_off, d_tokens, d_out, dim / 256u, vocab, ctx->d_flag);
    return lev_hip_check(ctx, hipGetLastError(), "embed_q4_k launch");
}

extern "C" int lev_hip_dequant(lev_ctx *ctx, int type, const void *d_w, size_t w_bytes,
                               uint64_t w_off, uint64_t nblocks, float *d_out,
                               size_t out_capacity) {
    LEV_REQUIRE_CTX(ctx);
    if (!d_w || !d_out) return lev_fail(ctx, LEV_ERR_INVALID_ARGUMENT, "dequant: null pointer");
    uint32_t bytes, values;
    switch (type) {
        case LEV_TYPE_Q4_0: bytes = 18; values = 32; break;
        case LEV_TYPE_Q4_K: bytes = 144; values = 256; break;
        case LEV_TYPE_Q6_K: bytes = 210; values = 256; break;
        default: return lev_fail(ctx, LEV_ERR_BAD_DIMENSIONS, "dequant: unsupported type %d", type);
    }
    uint64_t need, end, nvalues;
    if (nblocks == 0) return lev_fail(ctx, LEV_ERR_BAD_DIMENSIONS, "dequant: 0 blocks");
    if (__builtin_mul_overflow(nblocks, (uint64_t)bytes, &need) ||
        __builtin_add_overflow(w_off, need, &end) ||
        __builtin_mul_overflow(nblocks, (uint64_t)values, &nvalues))
        return lev_fail(ctx, LEV_ERR_INTEGER_OVERFLOW, "dequant: extent overflows");
    if (end > w_bytes || need > LEV_MAX_Q4_WEIGHT_BYTES)
        return lev_fail(ctx, LEV_ERR_BAD_DIMENSIONS, "dequant: blocks [%llu, %llu) beyond %zu bytes",
                        (unsigned long long)w_off, (unsigned long long)end, w_bytes);
    if (out_capacity < nvalues)
        return lev_fail(ctx, LEV_ERR_BAD_DIMENSIONS, "dequant: out holds %zu, needs %llu",
                        out_capacity, (unsigned long long)nvalues);
    const uint8_t *w = static_cast<const uint8_t *>(d_w) + w_off;
    uint64_t groups = (nvalues + 255) / 256;
    if (groups > 0x7FFFFFFFull) return lev_fail(ctx, LEV_ERR_EXCEEDS_MODEL_WORKLOAD, "dequant: grid");
    dim3 grid((unsigned)groups), block(256);
    if (type == LEV_TYPE_Q4_0)
        hipLaunchKernelGGL(dequant_q4_0, grid, block, 0, ctx->stream, w, d_out, nvalues);
    else if (type == LEV_TYPE_Q6_K)
        hipLaunchKernelGGL(dequant_q6_k, grid, block, 0, ctx->stream, w, d_out, nvalues);
    else
        hipLaunchKernelGGL(dequant_q4_k, grid, block, 0, ctx->stream, w, d_out, nvalues);
    return lev_hip_check(ctx, hipGetLastError(), "dequant launch");
}

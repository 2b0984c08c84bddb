// Q4_0 device primitives shared by the decode GEMV and the MoE expert kernels.
//
// Data layout in HBM is the GGUF one, untouched: 18-byte blocks (fp16 d,
// 16 code bytes; byte l low nibble -> element l, high nibble -> element 16+l,
// w = d*(n-8); Q4.swift:33-69).  A row of in_dim values is in_dim/32
// consecutive blocks; rows follow each other with no padding.
//
// Work unit of every kernel here: a PAIR of adjacent blocks = 36 bytes, which
// is 4-byte aligned whenever the row is (rows of an even number of blocks
// always are), so a lane fetches a pair with two 128-bit loads and one 32-bit
// load, and the 64 lanes of a wave fetch 2304 contiguous bytes.
//
// A lane keeps the 64 activations of its pair in registers (16 x float4) and
// reuses them for every row it visits.  The -8 offset is folded out of the
// inner loop:  sum_l d*(n_l-8)*x_l = d*(sum_l n_l*x_l - 8*sum_l x_l).
#pragma once

#include "lev_common.hpp"

#ifndef LEV_Q4_MIX
// 1: nibbles become fp16 subnormals (n * 2^-24) with one AND per two weights
//    and feed v_fma_mix_f32 directly; 0: v_cvt_f32_ubyteN per weight.
#define LEV_Q4_MIX 1
#endif

// Activations of one pair: xr[q] holds elements 4q..4q+3 of the 64.
struct lev_q4_pair_x {
    lev_f32x4 xr[16];
    float sum_a;   // sum of elements 0..31   (first block)
    float sum_b;   // sum of elements 32..63  (second block)
};

__device__ __forceinline__ void lev_q4_pair_x_sums(lev_q4_pair_x &px) {
    float a0 = 0.f, a1 = 0.f, b0 = 0.f, b1 = 0.f;
#pragma unroll
    for (int q = 0; q < 8; q += 2) {
        a0 += (px.xr[q].x + px.xr[q].y) + (px.xr[q].z + px.xr[q].w);
        a1 += (px.xr[q + 1].x + px.xr[q + 1].y) + (px.xr[q + 1].z + px.xr[q + 1].w);
        b0 += (px.xr[8 + q].x + px.xr[8 + q].y) + (px.xr[8 + q].z + px.xr[8 + q].w);
        b1 += (px.xr[9 + q].x + px.xr[9 + q].y) + (px.xr[9 + q].z + px.xr[9 + q].w);
    }
    px.sum_a = a0 + a1;
    px.sum_b = b0 + b1;
}

// sum over the 32 weights of one block of n_l * x_l, with the block's 16 code
// bytes in q[0..3] (byte l = code byte l) and its activations in x[0..7]
// (x[j] = elements 4j..4j+3).  Returns the sum scaled by `scale_out`:
//   LEV_Q4_MIX: result * 2^-24 (caller multiplies d by 2^24)
template <int MIX>
__device__ __forceinline__ float lev_q4_block_dot(const uint32_t q[4], const lev_f32x4 *x);

template <>
__device__ __forceinline__ float lev_q4_block_dot<0>(const uint32_t q[4], const lev_f32x4 *x) {
    float lo = 0.f, hi = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        uint32_t l4 = q[j] & 0x0F0F0F0Fu;
        uint32_t h4 = (q[j] >> 4) & 0x0F0F0F0Fu;
        lev_f32x4 xl = x[j], xh = x[4 + j];
        lo = fmaf((float)(l4 & 0xFF), xl.x, lo);
        lo = fmaf((float)((l4 >> 8) & 0xFF), xl.y, lo);
        lo = fmaf((float)((l4 >> 16) & 0xFF), xl.z, lo);
        lo = fmaf((float)(l4 >> 24), xl.w, lo);
        hi = fmaf((float)(h4 & 0xFF), xh.x, hi);
        hi = fmaf((float)((h4 >> 8) & 0xFF), xh.y, hi);
        hi = fmaf((float)((h4 >> 16) & 0xFF), xh.z, hi);
        hi = fmaf((float)(h4 >> 24), xh.w, hi);
    }
    return lo + hi;
}

template <>
__device__ __forceinline__ float lev_q4_block_dot<1>(const uint32_t q[4], const lev_f32x4 *x) {
    // fp16 bit pattern 0x000n is the subnormal n*2^-24 and 0x00n0 is 16n*2^-24:
    // both convert to f32 exactly, so masking IS the dequantisation.
    float lo = 0.f, hi = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        uint32_t w = q[j], s = w >> 8;
        lev_f16x2 l02 = __builtin_bit_cast(lev_f16x2, w & 0x000F000Fu);   // bytes 0,2 low
        lev_f16x2 h02 = __builtin_bit_cast(lev_f16x2, w & 0x00F000F0u);   // bytes 0,2 high (x16)
        lev_f16x2 l13 = __builtin_bit_cast(lev_f16x2, s & 0x000F000Fu);   // bytes 1,3 low
        lev_f16x2 h13 = __builtin_bit_cast(lev_f16x2, s & 0x00F000F0u);   // bytes 1,3 high (x16)
        lev_f32x4 xl = x[j], xh = x[4 + j];
        lo = fmaf((float)l02.x, xl.x, lo);
        lo = fmaf((float)l13.x, xl.y, lo);
        lo = fmaf((float)l02.y, xl.z, lo);
        lo = fmaf((float)l13.y, xl.w, lo);
        hi = fmaf((float)h02.x, xh.x, hi);
        hi = fmaf((float)h13.x, xh.y, hi);
        hi = fmaf((float)h02.y, xh.z, hi);
        hi = fmaf((float)h13.y, xh.w, hi);
    }
    return fmaf(hi, 0.0625f, lo);
}

// Contribution of one pair (36 bytes in D[0..8], little-endian dwords from a
// 4-byte aligned address) to its row's dot product.
__device__ __forceinline__ float lev_q4_pair_dot(const uint32_t D[9], const lev_q4_pair_x &px) {
    float da = lev_f16_bits_to_f32(D[0] & 0xFFFFu);
    float db = lev_f16_bits_to_f32(D[4] >> 16);
    uint32_t qa[4], qb[4];
    qa[0] = __builtin_amdgcn_alignbit(D[1], D[0], 16);
    qa[1] = __builtin_amdgcn_alignbit(D[2], D[1], 16);
    qa[2] = __builtin_amdgcn_alignbit(D[3], D[2], 16);
    qa[3] = __builtin_amdgcn_alignbit(D[4], D[3], 16);
    qb[0] = D[5];
    qb[1] = D[6];
    qb[2] = D[7];
    qb[3] = D[8];
    float sa = lev_q4_block_dot<LEV_Q4_MIX>(qa, &px.xr[0]);
    float sb = lev_q4_block_dot<LEV_Q4_MIX>(qb, &px.xr[8]);
#if LEV_Q4_MIX
    sa *= 16777216.0f;
    sb *= 16777216.0f;
#endif
    return fmaf(da, fmaf(-8.0f, px.sum_a, sa), db * fmaf(-8.0f, px.sum_b, sb));
}

// Loads a pair.  `p` points at the pair's first byte (4-byte aligned).
__device__ __forceinline__ void lev_q4_load_pair(const uint8_t *p, uint32_t D[9]) {
    lev_u32x4_a4 a = *reinterpret_cast<const lev_u32x4_a4 *>(p);
    lev_u32x4_a4 b = *reinterpret_cast<const lev_u32x4_a4 *>(p + 16);
    lev_u32_a4 c = *reinterpret_cast<const lev_u32_a4 *>(p + 32);
    D[0] = a.v[0]; D[1] = a.v[1]; D[2] = a.v[2]; D[3] = a.v[3];
    D[4] = b.v[0]; D[5] = b.v[1]; D[6] = b.v[2]; D[7] = b.v[3];
    D[8] = c.v;
}

__device__ __forceinline__ void lev_q4_zero_pair(uint32_t D[9]) {
#pragma unroll
    for (int i = 0; i < 9; ++i) D[i] = 0u;
}

// Stages a vector of n floats (n a multiple of 64) into LDS in the pair-major
// transposed layout: float4 slot q*(P+1)+p holds elements 64p+4q..64p+4q+3,
// so that lanes owning consecutive pairs read consecutive 16-byte slots.
// Split in two so that callers can put other global loads between the load
// and the store: the loads are issued first (they are short and usually hit
// L2), the caller's weight loads follow, and the wait for the activations
// does not have to wait for the weights (VMEM returns in issue order).
constexpr int kLevStageSlots = 4;   // default number of float4 per thread covered in registers

// FULL: the caller guarantees pairs*16 == NS*nthreads (every slot in range,
// nothing beyond), which removes every bounds test from the staging code.
template <int NS = kLevStageSlots, bool FULL = false>
__device__ __forceinline__ void lev_q4_stage_x_load(const float *__restrict__ x, uint32_t pairs,
                                                    uint32_t tid, uint32_t nthreads,
                                                    lev_f32x4 v[NS]) {
    const lev_f32x4 *x4 = reinterpret_cast<const lev_f32x4 *>(x);
    const uint32_t n4 = pairs * 16u;
    if (FULL) {
#pragma unroll
        for (int k = 0; k < NS; ++k) v[k] = x4[tid + k * nthreads];
        return;
    }
    // Unconditional loads from clamped indices: a branch around a load makes
    // the compiler wait for every outstanding load at the join, which would
    // serialise these four.
#pragma unroll
    for (int k = 0; k < NS; ++k) {
        uint32_t i = tid + k * nthreads;
        v[k] = x4[i < n4 ? i : n4 - 1u];
    }
}

template <int NS = kLevStageSlots>
__device__ __forceinline__ void lev_q4_stage_x_store(const float *__restrict__ x, lev_f32x4 *xs,
                                                     uint32_t pairs, uint32_t tid,
                                                     uint32_t nthreads,
                                                     const lev_f32x4 v[NS]) {
    const lev_f32x4 *x4 = reinterpret_cast<const lev_f32x4 *>(x);
    const uint32_t n4 = pairs * 16u;
#pragma unroll
    for (int k = 0; k < NS; ++k) {
        uint32_t i = tid + k * nthreads;
        if (i < n4) xs[(i & 15u) * (pairs + 1u) + (i >> 4)] = v[k];
    }
    // vectors longer than NS*nthreads float4 (rare): the rest
    for (uint32_t i = tid + NS * nthreads; i < n4; i += nthreads)
        xs[(i & 15u) * (pairs + 1u) + (i >> 4)] = x4[i];
}

__device__ __forceinline__ void lev_q4_stage_x(const float *__restrict__ x, lev_f32x4 *xs,
                                               uint32_t pairs, uint32_t tid, uint32_t nthreads) {
    lev_f32x4 v[kLevStageSlots];
    lev_q4_stage_x_load<kLevStageSlots>(x, pairs, tid, nthreads, v);
    lev_q4_stage_x_store<kLevStageSlots>(x, xs, pairs, tid, nthreads, v);
}

// As lev_q4_stage_x_store, and also writes the sum of every block of 32
// activations to bsum[block] (a block is 8 consecutive float4, i.e. 8
// consecutive threads of one pass, so the sum is three DPP steps).  nthreads
// must be a multiple of 8.  bsum needs 2*pairs floats.
template <int NS = kLevStageSlots, bool FULL = false>
__device__ __forceinline__ void lev_q4_stage_x_store_sums(const float *__restrict__ x,
                                                          lev_f32x4 *xs, float *bsum,
                                                          uint32_t pairs, uint32_t tid,
                                                          uint32_t nthreads,
                                                          const lev_f32x4 v[NS]) {
    const lev_f32x4 *x4 = reinterpret_cast<const lev_f32x4 *>(x);
    const uint32_t n4 = pairs * 16u;
    if (FULL) {
#pragma unroll
        for (int k = 0; k < NS; ++k) {
            const uint32_t i = tid + k * nthreads;
            float s4 = (v[k].x + v[k].y) + (v[k].z + v[k].w);
            s4 = lev_group_sum<8>(s4);
            xs[(i & 15u) * (pairs + 1u) + (i >> 4)] = v[k];
            if ((i & 7u) == 7u) bsum[i >> 3] = s4;
        }
        return;
    }
    auto put = [&](uint32_t i, lev_f32x4 val) {
        float s4 = (val.x + val.y) + (val.z + val.w);
        s4 = lev_group_sum<8>(s4);
        if (i < n4) {
            xs[(i & 15u) * (pairs + 1u) + (i >> 4)] = val;
            if ((i & 7u) == 7u) bsum[i >> 3] = s4;
        }
    };
#pragma unroll
    for (int k = 0; k < NS; ++k) put(tid + k * nthreads, v[k]);
    const uint32_t covered = NS * nthreads;
    if (n4 > covered) {   // longer vectors: whole extra passes, every thread takes part in the DPP sums
        for (uint32_t base = covered; base < n4; base += nthreads) {
            uint32_t i = base + tid;
            put(i, x4[i < n4 ? i : n4 - 1u]);
        }
    }
}

// Fetches the activations of pair p with the block sums read from bsum.
__device__ __forceinline__ void lev_q4_fetch_x_sums(const lev_f32x4 *xs, const float *bsum,
                                                    uint32_t pairs, uint32_t p, lev_q4_pair_x &px) {
#pragma unroll
    for (int q = 0; q < 16; ++q) px.xr[q] = xs[q * (pairs + 1u) + p];
    px.sum_a = bsum[2u * p];
    px.sum_b = bsum[2u * p + 1u];
}

__device__ __forceinline__ void lev_q4_fetch_x(const lev_f32x4 *xs, uint32_t pairs, uint32_t p,
                                               lev_q4_pair_x &px) {
#pragma unroll
    for (int q = 0; q < 16; ++q) px.xr[q] = xs[q * (pairs + 1u) + p];
    lev_q4_pair_x_sums(px);
}

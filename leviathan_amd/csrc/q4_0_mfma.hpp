// Q4_0 x f32 on the integer matrix cores: the building block of the decode GEMV and of the
// MoE expert kernels at few tokens.
//
// One TASK is 16 weight rows x 4 pairs of blocks (256 activations).  v_mfma_i32_16x16x64_i8
// multiplies 16 rows x 64 codes; lane (r, g) = (lane % 16, lane / 16) supplies, as B, 16 codes of
// row r: the low nibbles, then the high nibbles, of one block of ITS OWN pair (pair 4T + g of the
// task), as int8 bytes 16*(n - 8) -- one bit operation per four codes: masking a nibble into the
// high half of a byte and flipping its top bit IS the signed value, so the offset of the format
// never needs a correction term.  A row 4g + p holds digit plane p of the 16 activations lane
// group g multiplies and zeros elsewhere (the other lanes read a zeroed strip), so accumulator
// register p of lane (r, g) is the plane-p sum of that lane's own codes: nothing is exchanged
// between lanes until a row's four lane groups add their finished pair sums.
//
// Activations: per pair of blocks (64 values) x becomes integers X = rint(x * 2^(156 - ex)),
// |X| <= 2^30, ex the biased exponent of the pair's largest magnitude: every value within 2^-6 of
// that maximum is represented exactly.  X is cut into four balanced base-256 digits (the bytes of
// (X + 0x808080) ^ 0x808080 read as int8).  The integer sums are exact; a block's planes are
// recombined and scaled by d in f32, so what is rounded is one number per block of 32 weights.
//
// A wave stages the 256 activations of its own task by itself (one float4 per lane, a 1 KB area
// of LDS nobody else touches): no workgroup barrier stands between the activations and the
// products, and the A operands (16 registers a task) serve every row group the wave visits.
//
// Weight bytes are fetched with the four pairs of a row in four ADJACENT lanes (lane = 4*row +
// pair: a quad reads 144 contiguous bytes; with lane = 16*pair + row every quad touches four
// rows and the same read of a cold 9 MB matrix takes 0.3 us longer) and handed to the lane the
// matrix core wants them in by one lane permutation per dword.
#pragma once

#include "q4_0_device.hpp"

typedef int lev_i32x4 __attribute__((ext_vector_type(4)));

constexpr uint32_t kLevQ4MfmaMaxInDim = 8192u;   // widest row the matrix-core GEMV takes
constexpr uint32_t kQ4mTaskArea = 1024u;   // LDS bytes of one staged task: [pair 4][plane 4][half 4][16 B]
constexpr uint32_t kQ4mZeroBytes = 16u;    // what the lanes outside a row's own lane group read as their A operand

// A operands of one task (four halves: block A low / high nibbles, block B low / high) and the
// power of two that undoes the scaling of the lane's own pair (and the 16 of the codes).
struct q4m_operand {
    lev_i32x4 a[4];
    float unscale;
};

// Stages the task whose activations are v (lane i holds elements 4i..4i+3 of the task's 256)
// into `area` (kQ4mTaskArea bytes, this wave's own) and reads the lane's A operands back.
// `zero` points at kQ4mZeroBytes of zeros.  live == false: the task lies beyond the row (its
// operands are zero, it adds nothing).  A NaN or an infinity among the 64 activations of a pair
// makes the pair's factor NaN, and with it every row's sum.
__device__ __forceinline__ void q4m_stage_task(const lev_f32x4 v, uint8_t *area, const uint8_t *zero,
                                               bool live, q4m_operand &op) {
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t r = lane & 15u, g = lane >> 4;
    uint32_t mb = 0u;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const uint32_t bits = __float_as_uint(v[k]) & 0x7FFFFFFFu;
        mb = bits > mb ? bits : mb;
    }
    mb = lev_row16_max_u32(mb);   // the 16 lanes of a pair hold the pair's maximum
    uint32_t ex = mb >> 23;                                    // |x| < 2^(ex - 126)
    const bool bad = ex == 255u;
    ex = ex < 34u ? 34u : (ex > 254u ? 254u : ex);             // keeps both powers of two normal numbers
    const float scale = __uint_as_float((283u - ex) << 23);    // 2^(156 - ex): |x * scale| < 2^30
    op.unscale = !live ? 0.f : bad ? __builtin_nanf("") : __uint_as_float((ex - 33u) << 23);   // 2^(ex - 160)
    uint32_t Y[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) Y[k] = ((uint32_t)(int)rintf(v[k] * scale) + 0x00808080u) ^ 0x00808080u;
    // 4x4 byte transpose: digit p of the lane's four values in one dword
    const uint32_t t0 = __builtin_amdgcn_perm(Y[1], Y[0], 0x05010400u);
    const uint32_t t1 = __builtin_amdgcn_perm(Y[1], Y[0], 0x07030602u);
    const uint32_t t2 = __builtin_amdgcn_perm(Y[3], Y[2], 0x05010400u);
    const uint32_t t3 = __builtin_amdgcn_perm(Y[3], Y[2], 0x07030602u);
    uint32_t dw[4];
    dw[0] = __builtin_amdgcn_perm(t2, t0, 0x05040100u);
    dw[1] = __builtin_amdgcn_perm(t2, t0, 0x07060302u);
    dw[2] = __builtin_amdgcn_perm(t3, t1, 0x05040100u);
    dw[3] = __builtin_amdgcn_perm(t3, t1, 0x07060302u);
    // lane i: pair i / 16, half (i % 16) / 4, k-slots 4 * (i % 4) .. + 3
    uint8_t *at = area + g * 256u + (r >> 2) * 16u + (r & 3u) * 4u;
#pragma unroll
    for (int p = 0; p < 4; ++p) *reinterpret_cast<uint32_t *>(at + 64 * p) = dw[p];
    // the area belongs to this wave alone: LDS runs a wave's accesses in order, the fences only
    // keep the compiler from moving the reads above the writes
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const bool feeds = live && (r >> 2) == g;                  // A row r belongs to lane group r / 4
    const uint8_t *ab = feeds ? area + g * 256u + (r & 3u) * 64u : zero;
    const uint32_t hs = feeds ? 16u : 0u;
#pragma unroll
    for (int h = 0; h < 4; ++h) op.a[h] = *reinterpret_cast<const lev_i32x4 *>(ab + h * hs);
}

// The weights of one task as they are fetched: lane 4*row + pair holds pair `pair` of row `row`.
// `rowp` = first byte of the lane's row (row lane / 4 of the group), task_pair0 = 4 * task.
__device__ __forceinline__ void q4m_load_task(const uint8_t *rowp, uint32_t task_pair0, uint32_t D[9]) {
    const uint32_t lane = threadIdx.x & 63u;
    lev_q4_load_pair(rowp + (uint64_t)(task_pair0 + (lane & 3u)) * 36u, D);
}

// Lane (r, g) <- lane 4*r + g, for every dword of a fetched task.
__device__ __forceinline__ void q4m_turn_task(const uint32_t D[9], uint32_t W[9]) {
    const uint32_t lane = threadIdx.x & 63u;
    const int src = (int)((4u * (lane & 15u) + (lane >> 4)) * 4u);
#pragma unroll
    for (int k = 0; k < 9; ++k) W[k] = (uint32_t)__builtin_amdgcn_ds_bpermute(src, (int)D[k]);
}

// Contribution of the lane's pair (W: its 36 bytes, already turned) to its row's dot product.
__device__ __forceinline__ float q4m_task_dot(const uint32_t W[9], const q4m_operand &op) {
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    const float da = lev_f16_bits_to_f32(W[0] & 0xFFFFu);
    const float db = lev_f16_bits_to_f32(W[4] >> 16);
    u4 qa, qb;
    qa.x = __builtin_amdgcn_alignbit(W[1], W[0], 16);
    qa.y = __builtin_amdgcn_alignbit(W[2], W[1], 16);
    qa.z = __builtin_amdgcn_alignbit(W[3], W[2], 16);
    qa.w = __builtin_amdgcn_alignbit(W[4], W[3], 16);
    qb = u4{W[5], W[6], W[7], W[8]};
    // int8 bytes 16*(n - 8): the nibble in the high half of its byte, its top bit flipped
    const lev_i32x4 bal = __builtin_bit_cast(lev_i32x4, ((qa << 4) & 0xF0F0F0F0u) ^ 0x80808080u);
    const lev_i32x4 bah = __builtin_bit_cast(lev_i32x4, (qa & 0xF0F0F0F0u) ^ 0x80808080u);
    const lev_i32x4 bbl = __builtin_bit_cast(lev_i32x4, ((qb << 4) & 0xF0F0F0F0u) ^ 0x80808080u);
    const lev_i32x4 bbh = __builtin_bit_cast(lev_i32x4, (qb & 0xF0F0F0F0u) ^ 0x80808080u);
    lev_i32x4 sa = __builtin_amdgcn_mfma_i32_16x16x64_i8(op.a[0], bal, lev_i32x4{0, 0, 0, 0}, 0, 0, 0);
    lev_i32x4 sb = __builtin_amdgcn_mfma_i32_16x16x64_i8(op.a[2], bbl, lev_i32x4{0, 0, 0, 0}, 0, 0, 0);
    sa = __builtin_amdgcn_mfma_i32_16x16x64_i8(op.a[1], bah, sa, 0, 0, 0);
    sb = __builtin_amdgcn_mfma_i32_16x16x64_i8(op.a[3], bbh, sb, 0, 0, 0);
    // |plane sum| <= 32 * 128 * 128 = 2^19: two planes recombine in 32 bits, the halves in f32
    const float fa = fmaf((float)(sa[2] + (sa[3] << 8)), 65536.0f, (float)(sa[0] + (sa[1] << 8)));
    const float fb = fmaf((float)(sb[2] + (sb[3] << 8)), 65536.0f, (float)(sb[0] + (sb[1] << 8)));
    return fmaf(da, fa, db * fb) * op.unscale;
}

// Sum over lanes l, l ^ 16, l ^ 32, l ^ 48 (the four lane groups of a row), in every lane,
// by two row swaps: no LDS.
__device__ __forceinline__ float q4m_row_sum(float v) {
    const uint32_t u = __float_as_uint(v);
    const auto s0 = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    v = __uint_as_float(s0[0]) + __uint_as_float(s0[1]);
    const uint32_t u2 = __float_as_uint(v);
    const auto s1 = __builtin_amdgcn_permlane16_swap(u2, u2, false, false);
    return __uint_as_float(s1[0]) + __uint_as_float(s1[1]);
}


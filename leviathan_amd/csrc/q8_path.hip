// Int8-activation decode path for gfx950: RMSNorm + int8 quantisation of the
// activations, and the Q4_K multi-column GEMV on integer dot products.
//
// Stands in for the reference's production decode kernels on Vulkan:
//   quantize             emit_quantize, rust/crates/lev-forge/src/q8.rs:20-51
//   (add +) rmsnorm + quantize (+ f32 out)
//                        emit_norm_quant / QUANT_STEP, lev-forge/src/q8.rs:105-164
//                        (CPU statement: quantize_q8, rust/crates/lev-cpu/src/lib.rs:295-322)
//   q4k.q8.matvec        rust/crates/lev-forge/src/q8.rs:196-326, nb columns per weight read
//                        (oracle: matvec_q4k_q8_f64, lev-cpu/src/lib.rs:324-331)
//
// Activations: groups of 32, d = amax/127, q = round_half_even(x * (127/amax)),
// s = d * sum(q).  xq holds the int8 codes (4 per dword, element order), xs the
// (d, s) pair of each group.
//
// GEMV, per superblock of a row (w = d*sc_j*q - dmin*m_j, a sub-block of 32
// weights lines up with one activation group):
//   y += d * sum_j sc_j * dx_j * (sum_l q_l * xq_l)  -  dmin * sum_j m_j * s_j
// The inner sum is exact in int32: v_dot4_i32_i8 on the nibbles (unpacked to
// bytes with one AND per four weights) against the activation codes.  About
// 0.6 vector instructions per weight and column, so the kernel stays HBM-bound
// for the column counts of speculative verify.
#include "lev_common.hpp"

#include <cstdlib>

#pragma clang fp contract(off)

namespace {

// ---------------------------------------------------------------------------
// RMSNorm (optional) + quantize.  One workgroup of 1024 threads per column; a
// thread owns four consecutive values (one 16-byte load, one packed dword of
// codes), so a group of 32 is eight lanes and its maximum and code sum are
// three DPP steps each.
// With a gain the normalised value is formed as the reference CPU path does
// (f64 mean of squares, (float)(x * inv) * w, lev-model/src/lib.rs:110-114), so
// that the codes match quantize_q8(rmsnorm(x)) bit for bit.
// ---------------------------------------------------------------------------
constexpr int kNQThreads = 1024;
typedef float lev_f32x2 __attribute__((ext_vector_type(2)));

template <int CTRL>
__device__ __forceinline__ float dpp_max(float v) {
    int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true);
    return fmaxf(v, __builtin_bit_cast(float, moved));
}
template <int CTRL>
__device__ __forceinline__ int dpp_addi(int v) {
    return v + __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, true);
}

__global__ void __launch_bounds__(kNQThreads)
norm_quant_kernel(float *__restrict__ x, const float *__restrict__ add,
                  const float *__restrict__ gain, float eps, uint32_t *__restrict__ xq,
                  float *__restrict__ xs, float *__restrict__ y_out, uint32_t n) {
    __shared__ double s_part[kNQThreads / 64];
    const uint32_t col = blockIdx.x, t = threadIdx.x, lane = t & 63u;
    const uint32_t n4 = n >> 2;
    lev_f32x4 *xc = reinterpret_cast<lev_f32x4 *>(x + (uint64_t)col * n);
    const lev_f32x4 *gc = reinterpret_cast<const lev_f32x4 *>(gain);
    // The first pass keeps its values in registers (every column of up to 4096
    // values is one pass); later passes reread their own elements.
    lev_f32x4 first = {0.f, 0.f, 0.f, 0.f};
    double inv = 1.0;
    if (add || gain) {
        const lev_f32x4 *ac = reinterpret_cast<const lev_f32x4 *>(add + (add ? (uint64_t)col * n : 0));
        double ss = 0.0;
        for (uint32_t i = t; i < n4; i += kNQThreads) {
            lev_f32x4 v = xc[i];
            if (add) {   // residual add first, written back (x += d, q8.rs:152-154)
                const lev_f32x4 a = ac[i];
                v.x = v.x + a.x, v.y = v.y + a.y, v.z = v.z + a.z, v.w = v.w + a.w;
                xc[i] = v;
            }
            if (i == t) first = v;
            ss += (double)v.x * (double)v.x;
            ss += (double)v.y * (double)v.y;
            ss += (double)v.z * (double)v.z;
            ss += (double)v.w * (double)v.w;
        }
        if (gain) {
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off);
            if (lane == 0) s_part[t >> 6] = ss;
            lev_barrier_lds();
            double tot = 0.0;
#pragma unroll
            for (int k = 0; k < kNQThreads / 64; ++k) tot += s_part[k];
            inv = 1.0 / sqrt(tot / (double)n + (double)eps);
        }
    } else if (t < n4) {
        first = xc[t];
    }
    // whole passes: every lane takes part in the group reductions
    for (uint32_t base = 0; base < n4; base += kNQThreads) {
        const uint32_t i = base + t;
        const bool live = i < n4;          // n % 32 == 0: the eight lanes of a group are live or not together
        lev_f32x4 v = first;
        if (base != 0u) {
            v = lev_f32x4{0.f, 0.f, 0.f, 0.f};
            if (live) v = xc[i];
        }
        if (gain && live) {
            const lev_f32x4 g = gc[i];
            v.x = (float)((double)v.x * inv) * g.x;
            v.y = (float)((double)v.y * inv) * g.y;
            v.z = (float)((double)v.z * inv) * g.z;
            v.w = (float)((double)v.w * inv) * g.w;
        }
        if (y_out && live) reinterpret_cast<lev_f32x4 *>(y_out + (uint64_t)col * n)[i] = v;
        float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
        amax = dpp_max<0xB1>(amax);        // quad_perm [1,0,3,2]
        amax = dpp_max<0x4E>(amax);        // quad_perm [2,3,0,1]
        amax = dpp_max<0x141>(amax);       // row_half_mirror: all eight lanes hold the group's maximum
        const float dq = amax / 127.0f;
        const float idq = amax > 0.0f ? 127.0f / amax : 0.0f;
        const int q0 = (int)rintf(v.x * idq), q1 = (int)rintf(v.y * idq);   // round half to even
        const int q2 = (int)rintf(v.z * idq), q3 = (int)rintf(v.w * idq);
        int qsum = (q0 + q1) + (q2 + q3);
        qsum = dpp_addi<0xB1>(qsum);
        qsum = dpp_addi<0x4E>(qsum);
        qsum = dpp_addi<0x141>(qsum);
        if (live) {
            xq[(uint64_t)col * n4 + i] = ((uint32_t)q0 & 255u) | (((uint32_t)q1 & 255u) << 8) |
                                         (((uint32_t)q2 & 255u) << 16) | ((uint32_t)q3 << 24);
            if ((t & 7u) == 0u) {
                lev_f32x2 pair = {dq, dq * (float)qsum};
                reinterpret_cast<lev_f32x2 *>(xs)[((uint64_t)col * n4 + i) >> 3] = pair;
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Q4_K x int8 GEMV, NC columns.  Workgroup = 4 waves; 16 lanes per row (a lane
// owns whole superblocks: sb = lane%16, +16, ...), so a wave covers 4 rows and
// its loads read those rows contiguously.
// LDS: activation codes [col][sb] padded to 272 B, (d, s) pairs [col][sb] padded
// to 80 B (both strides spread the 16 lanes of a row over the banks).
// ---------------------------------------------------------------------------
// workgroup sizes as measured: four waves for the Q4_K kernel (12288x4096, one column: 8.6 us
// against 10.1 with eight), eight for the Q6_K kernel (32000x4096, eight columns: 40.7 against 42.5)
constexpr int kQThreads = 256;
constexpr int kQ6Threads = 512;
constexpr uint32_t kQ4Rows = (kQThreads / 64) * 4;    // rows per workgroup tile, Q4_K kernel (16 lanes a row)
constexpr uint32_t kQ6Rows = (kQ6Threads / 64) * 2;   // Q6_K kernel (32 lanes a row)
constexpr uint32_t kCodeStride = 272, kPairStride = 80;

struct q4k_block_regs {
    lev_u32x4 hdr;
    lev_u32x4 qs[8];
};

__device__ __forceinline__ void q8_issue(const uint8_t *__restrict__ p, q4k_block_regs &b) {
    b.hdr = *reinterpret_cast<const lev_u32x4 *>(p);
#pragma unroll
    for (int k = 0; k < 8; ++k) b.qs[k] = *reinterpret_cast<const lev_u32x4 *>(p + 16 + 16 * k);
}

template <int NC>
__global__ void __launch_bounds__(kQThreads)
q4_k_gemv_q8_kernel(const uint8_t *__restrict__ w, const uint32_t *__restrict__ xq,
                    const float *__restrict__ xs, float *__restrict__ y, uint32_t in_dim,
                    uint32_t rows, uint32_t ncol) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const uint32_t SB = in_dim >> 8;
    uint8_t *s_codes = smem;                                   // [NC][SB][272]
    uint8_t *s_pairs = smem + (size_t)NC * SB * kCodeStride;   // [NC][SB][80]
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;

    // stage the activations of every column (16-byte pieces)
    for (uint32_t i = tid; i < (uint32_t)NC * SB * 16u; i += kQThreads) {
        const uint32_t c = i / (SB * 16u), rem = i - c * (SB * 16u), sb = rem >> 4, k = rem & 15u;
        lev_u32x4 v = {0u, 0u, 0u, 0u};
        if (c < ncol) v = *reinterpret_cast<const lev_u32x4 *>(xq + ((uint64_t)c * in_dim >> 2) + sb * 64u + k * 4u);
        *reinterpret_cast<lev_u32x4 *>(s_codes + ((size_t)c * SB + sb) * kCodeStride + k * 16u) = v;
    }
    for (uint32_t i = tid; i < (uint32_t)NC * SB * 4u; i += kQThreads) {
        const uint32_t c = i / (SB * 4u), rem = i - c * (SB * 4u), sb = rem >> 2, k = rem & 3u;
        lev_f32x4 v = {0.f, 0.f, 0.f, 0.f};
        if (c < ncol) v = *reinterpret_cast<const lev_f32x4 *>(xs + ((uint64_t)c * (in_dim >> 5) + sb * 8u) * 2u + k * 4u);
        *reinterpret_cast<lev_f32x4 *>(s_pairs + ((size_t)c * SB + sb) * kPairStride + k * 16u) = v;
    }
    lev_barrier_lds();

    const uint32_t grp = lane >> 4, lp = lane & 15u;
    const uint64_t row_bytes = (uint64_t)SB * 144u;
    const uint32_t tiles = (rows + kQ4Rows - 1u) / kQ4Rows;
    for (uint32_t tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
        const uint32_t row = tile * kQ4Rows + wave * 4u + grp;
        const uint32_t rowc = row < rows ? row : rows - 1u;
        float acc[NC];
#pragma unroll
        for (int c = 0; c < NC; ++c) acc[c] = 0.f;
        for (uint32_t sb0 = 0; sb0 < SB; sb0 += 16u) {
            const uint32_t sb = sb0 + lp;
            const bool live = sb < SB;
            q4k_block_regs B;
            q8_issue(w + rowc * row_bytes + (uint64_t)(live ? sb : SB - 1u) * 144u, B);
            const float d = live ? lev_f16_bits_to_f32(B.hdr.x & 0xFFFFu) : 0.f;
            const float dmin = live ? lev_f16_bits_to_f32(B.hdr.x >> 16) : 0.f;
            const uint32_t S0 = B.hdr.y, S1 = B.hdr.z, S2 = B.hdr.w;
            float scf[8], mnf[8];   // unpack_scale_min, lev-cpu/src/lib.rs:64-74
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                scf[j] = (float)((S0 >> (8 * j)) & 63u);
                mnf[j] = (float)((S1 >> (8 * j)) & 63u);
                scf[4 + j] = (float)(((S2 >> (8 * j)) & 0xFu) | (((S0 >> (8 * j + 6)) & 3u) << 4));
                mnf[4 + j] = (float)(((S2 >> (8 * j + 4)) & 0xFu) | (((S1 >> (8 * j + 6)) & 3u) << 4));
            }
            const uint32_t sbc = live ? sb : SB - 1u;
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                const uint8_t *codes = s_codes + ((size_t)c * SB + sbc) * kCodeStride;
                const float *pairs = reinterpret_cast<const float *>(s_pairs + ((size_t)c * SB + sbc) * kPairStride);
                float a1 = 0.f, a2 = 0.f;
#pragma unroll
                for (int ch = 0; ch < 4; ++ch) {          // chunk: 32 code bytes, sub-blocks 2ch (low), 2ch+1 (high)
                    int lo = 0, hi = 0;
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        const lev_u32x4 q4 = B.qs[2 * ch + h];
                        const lev_u32x4 xl = *reinterpret_cast<const lev_u32x4 *>(codes + 64 * ch + 16 * h);
                        const lev_u32x4 xh = *reinterpret_cast<const lev_u32x4 *>(codes + 64 * ch + 32 + 16 * h);
#pragma unroll
                        for (int k = 0; k < 4; ++k) {
                            lo = __builtin_amdgcn_sdot4((int)(q4[k] & 0x0F0F0F0Fu), (int)xl[k], lo, false);
                            hi = __builtin_amdgcn_sdot4((int)((q4[k] >> 4) & 0x0F0F0F0Fu), (int)xh[k], hi, false);
                        }
                    }
                    const lev_f32x4 ds = *reinterpret_cast<const lev_f32x4 *>(pairs + 4 * ch);   // d, s of groups 2ch, 2ch+1
                    a1 = fmaf(scf[2 * ch] * ds.x, (float)lo, a1);
                    a1 = fmaf(scf[2 * ch + 1] * ds.z, (float)hi, a1);
                    a2 = fmaf(mnf[2 * ch], ds.y, a2);
                    a2 = fmaf(mnf[2 * ch + 1], ds.w, a2);
                }
                acc[c] = fmaf(d, a1, fmaf(-dmin, a2, acc[c]));
            }
        }
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            const float sum = lev_group_sum<16>(acc[c]);
            if (lp == 15u && row < rows && (uint32_t)c < ncol) y[(uint64_t)c * rows + row] = sum;
        }
    }
}

template <int NC>
hipError_t launch_q8(lev_ctx *ctx, const uint8_t *w, const uint32_t *xq, const float *xs, float *y,
                     uint32_t in_dim, uint32_t rows, uint32_t ncol) {
    const uint32_t SB = in_dim >> 8;
    const size_t lds = (size_t)NC * SB * (kCodeStride + kPairStride);
    static size_t configured = 0;
    if (lds > 48 * 1024 && lds > configured) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&q4_k_gemv_q8_kernel<NC>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        configured = lds;
    }
    int per_cu = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, q4_k_gemv_q8_kernel<NC>, kQThreads, lds) !=
            hipSuccess || per_cu < 1)
        per_cu = 1;
    const uint32_t tiles = (rows + kQ4Rows - 1u) / kQ4Rows;
    uint32_t blocks = (uint32_t)ctx->num_cus * (uint32_t)per_cu;
    if (blocks > tiles) blocks = tiles;
    hipLaunchKernelGGL((q4_k_gemv_q8_kernel<NC>), dim3(blocks), dim3(kQThreads), lds, ctx->stream, w, xq,
                       xs, y, in_dim, rows, ncol);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// Q6_K x int8 GEMV, NC columns (q6k.q8.matvec, emit_q6k_q8, lev-forge/src/q8.rs:330-447;
// oracle matvec_q6k_q8_f64, lev-cpu/src/lib.rs:333-337).
//
// A lane owns half a superblock: 64 ql bytes, the 32 qh bytes they pair with,
// 8 sub-scales and d (q6k_unpack, lev-cpu/src/lib.rs:203-216).  Its 128 weights
// are four activation groups of 32 (k = 0..3): byte l of the assembled dwords
//   k=0: (qlA & 15) | (qh     & 3) << 4      k=1: (qlB & 15) | (qh >> 2 & 3) << 4
//   k=2: (qlA >> 4) | (qh >> 4 & 3) << 4     k=3: (qlB >> 4) | (qh >> 6 & 3) << 4
// is element 32k + l, in the order of the activation codes, so every dword goes
// straight into v_dot4.  The codes stay unsigned (0..63); the -32 is applied
// through the sum of the activation codes over each 16 weights, formed once
// per column while staging:  sc * dx * (sum q*xq - 32 * sum xq).
// 32 lanes per row (4096 columns = 32 halves), a wave covers two rows.
// LDS per (column, superblock): 272 B of codes, 8 group scales, 16 code sums.
// ---------------------------------------------------------------------------
constexpr uint32_t kQ6Stride = 272 + 32 + 64;
struct __attribute__((packed, aligned(2))) q8_u32x4_a2 { uint32_t v[4]; };
struct __attribute__((packed, aligned(2))) q8_u32x2_a2 { uint32_t v[2]; };

template <int NC>
__global__ void __launch_bounds__(kQ6Threads)
q6_k_gemv_q8_kernel(const uint8_t *__restrict__ w, const uint32_t *__restrict__ xq,
                    const float *__restrict__ xs, float *__restrict__ y, uint32_t in_dim,
                    uint32_t rows, uint32_t ncol) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const uint32_t SB = in_dim >> 8;
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;

    // stage: 16-byte pieces of codes and their sums; group scales
    for (uint32_t i = tid; i < (uint32_t)NC * SB * 16u; i += kQ6Threads) {
        const uint32_t c = i / (SB * 16u), rem = i - c * (SB * 16u), sb = rem >> 4, k = rem & 15u;
        lev_u32x4 v = {0u, 0u, 0u, 0u};
        if (c < ncol) v = *reinterpret_cast<const lev_u32x4 *>(xq + ((uint64_t)c * in_dim >> 2) + sb * 64u + k * 4u);
        uint8_t *base = smem + ((size_t)c * SB + sb) * kQ6Stride;
        *reinterpret_cast<lev_u32x4 *>(base + k * 16u) = v;
        int sum = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) sum = __builtin_amdgcn_sdot4(0x01010101, (int)v[j], sum, false);
        reinterpret_cast<int *>(base + 304u)[k] = sum;
    }
    for (uint32_t i = tid; i < (uint32_t)NC * SB * 8u; i += kQ6Threads) {
        const uint32_t c = i / (SB * 8u), rem = i - c * (SB * 8u), sb = rem >> 3, k = rem & 7u;
        float d = 0.f;
        if (c < ncol) d = xs[((uint64_t)c * (in_dim >> 5) + sb * 8u + k) * 2u];
        reinterpret_cast<float *>(smem + ((size_t)c * SB + sb) * kQ6Stride + 272u)[k] = d;
    }
    lev_barrier_lds();

    const uint32_t grp = lane >> 5, lp = lane & 31u;
    const uint32_t halves = SB * 2u;
    const uint64_t row_bytes = (uint64_t)SB * 210u;
    const uint32_t tiles = (rows + kQ6Rows - 1u) / kQ6Rows;
    for (uint32_t tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
        const uint32_t row = tile * kQ6Rows + wave * 2u + grp;
        const uint32_t rowc = row < rows ? row : rows - 1u;
        float acc[NC];
#pragma unroll
        for (int c = 0; c < NC; ++c) acc[c] = 0.f;
        for (uint32_t h0 = 0; h0 < halves; h0 += 32u) {
            const uint32_t hh = h0 + lp;
            const bool live = hh < halves;
            const uint32_t hc = live ? hh : halves - 1u;
            const uint32_t sb = hc >> 1, half = hc & 1u;
            const uint8_t *blk = w + rowc * row_bytes + (uint64_t)sb * 210u;
            uint32_t qa[8], qb[8], qh[8];
#pragma unroll
            for (int k = 0; k < 2; ++k) {
                const q8_u32x4_a2 a = *reinterpret_cast<const q8_u32x4_a2 *>(blk + 64u * half + 16u * k);
                const q8_u32x4_a2 b = *reinterpret_cast<const q8_u32x4_a2 *>(blk + 64u * half + 32u + 16u * k);
                const q8_u32x4_a2 t = *reinterpret_cast<const q8_u32x4_a2 *>(blk + 128u + 32u * half + 16u * k);
#pragma unroll
                for (int j = 0; j < 4; ++j) qa[4 * k + j] = a.v[j], qb[4 * k + j] = b.v[j], qh[4 * k + j] = t.v[j];
            }
            const q8_u32x2_a2 scb = *reinterpret_cast<const q8_u32x2_a2 *>(blk + 192u + 8u * half);
            const float d = live ? lev_f16_bits_to_f32(*reinterpret_cast<const uint16_t *>(blk + 208u)) : 0.f;
            float scl[8];   // d * sub-scale: index 2k + p for group k, 16-weight part p
#pragma unroll
            for (int j = 0; j < 8; ++j)
                scl[j] = d * (float)(int)__builtin_amdgcn_sbfe((int)scb.v[j >> 2], 8 * (j & 3), 8);
            // the four code planes, eight dwords each
            uint32_t cw[4][8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                cw[0][i] = (qa[i] & 0x0F0F0F0Fu) | ((qh[i] << 4) & 0x30303030u);
                cw[1][i] = (qb[i] & 0x0F0F0F0Fu) | ((qh[i] << 2) & 0x30303030u);
                cw[2][i] = ((qa[i] >> 4) & 0x0F0F0F0Fu) | (qh[i] & 0x30303030u);
                cw[3][i] = ((qb[i] >> 4) & 0x0F0F0F0Fu) | ((qh[i] >> 2) & 0x30303030u);
            }
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                const uint8_t *base = smem + ((size_t)c * SB + sb) * kQ6Stride;
                const lev_f32x4 dx = *reinterpret_cast<const lev_f32x4 *>(base + 272u + 16u * half);
                float a = 0.f;
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const lev_u32x4 x0 = *reinterpret_cast<const lev_u32x4 *>(base + 128u * half + 32u * k);
                    const lev_u32x4 x1 = *reinterpret_cast<const lev_u32x4 *>(base + 128u * half + 32u * k + 16u);
                    const lev_u32x2 sums = *reinterpret_cast<const lev_u32x2 *>(base + 304u + 32u * half + 8u * k);
                    int lo = 0, hi = 0;
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        lo = __builtin_amdgcn_sdot4((int)cw[k][j], (int)x0[j], lo, false);
                        hi = __builtin_amdgcn_sdot4((int)cw[k][4 + j], (int)x1[j], hi, false);
                    }
                    lo -= 32 * (int)sums.x;
                    hi -= 32 * (int)sums.y;
                    a = fmaf(scl[2 * k] * dx[k], (float)lo, a);
                    a = fmaf(scl[2 * k + 1] * dx[k], (float)hi, a);
                }
                acc[c] += a;
            }
        }
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            const float sum = lev_group_sum<32>(acc[c]);
            if (lp == 31u && row < rows && (uint32_t)c < ncol) y[(uint64_t)c * rows + row] = sum;
        }
    }
}

template <int NC>
hipError_t launch_q6_q8(lev_ctx *ctx, const uint8_t *w, const uint32_t *xq, const float *xs, float *y,
                        uint32_t in_dim, uint32_t rows, uint32_t ncol, bool persistent) {
    const size_t lds = (size_t)NC * (in_dim >> 8) * kQ6Stride;
    static size_t configured = 0;
    if (lds > 48 * 1024 && lds > configured) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&q6_k_gemv_q8_kernel<NC>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        configured = lds;
    }
    int per_cu = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, q6_k_gemv_q8_kernel<NC>, kQ6Threads, lds) !=
            hipSuccess || per_cu < 1)
        per_cu = 1;
    const uint32_t tiles = (rows + kQ6Rows - 1u) / kQ6Rows;
    uint32_t blocks = (uint32_t)ctx->num_cus * (uint32_t)per_cu;
    if (blocks > tiles || !persistent) blocks = tiles;
    hipLaunchKernelGGL((q6_k_gemv_q8_kernel<NC>), dim3(blocks), dim3(kQ6Threads), lds, ctx->stream, w, xq,
                       xs, y, in_dim, rows, ncol);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// act = silu(gate) * up fused with the quantiser (emit_swiglu_quant,
// lev-forge/src/q8.rs:166-177; silu, lev-model/src/lib.rs:120).  Eight lanes of
// four values form a group of 32.
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(256)
swiglu_quant_kernel(const float *__restrict__ gate, const float *__restrict__ up, uint32_t *__restrict__ xq,
                    float *__restrict__ xs, float *__restrict__ act, uint32_t n4) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    const bool live = i < n4;                  // count % 32 == 0: eight lanes live or not together
    lev_f32x4 v = {0.f, 0.f, 0.f, 0.f};
    if (live) {
        const lev_f32x4 g = reinterpret_cast<const lev_f32x4 *>(gate)[i];
        const lev_f32x4 u = reinterpret_cast<const lev_f32x4 *>(up)[i];
#pragma unroll
        for (int k = 0; k < 4; ++k) v[k] = g[k] / (1.0f + expf(-g[k])) * u[k];
        if (act) reinterpret_cast<lev_f32x4 *>(act)[i] = v;
    }
    float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    amax = dpp_max<0xB1>(amax);
    amax = dpp_max<0x4E>(amax);
    amax = dpp_max<0x141>(amax);
    const float dq = amax / 127.0f;
    const float idq = amax > 0.0f ? 127.0f / amax : 0.0f;
    const int q0 = (int)rintf(v.x * idq), q1 = (int)rintf(v.y * idq);
    const int q2 = (int)rintf(v.z * idq), q3 = (int)rintf(v.w * idq);
    int qsum = (q0 + q1) + (q2 + q3);
    qsum = dpp_addi<0xB1>(qsum);
    qsum = dpp_addi<0x4E>(qsum);
    qsum = dpp_addi<0x141>(qsum);
    if (live) {
        xq[i] = ((uint32_t)q0 & 255u) | (((uint32_t)q1 & 255u) << 8) | (((uint32_t)q2 & 255u) << 16) |
                ((uint32_t)q3 << 24);
        if ((threadIdx.x & 7u) == 0u) {
            lev_f32x2 pair = {dq, dq * (float)qsum};
            reinterpret_cast<lev_f32x2 *>(xs)[i >> 3] = pair;
        }
    }
}

// ---------------------------------------------------------------------------
// Q4_K x int8 GEMV on the matrix cores, up to 16 columns per weight read.
//
// v_mfma_i32_16x16x32_i8, one per sub-block of 32 weights: A = the activation
// codes (16 "rows" = columns of x), B = 16 weight rows x 32 nibbles unpacked to
// bytes, exact int32 out.  Lane (r, g) = (l % 16, l / 16) loads row r's header
// and bytes 8g..8g+7 of each 32-byte chunk: their low nibbles are its 8 k-slots
// of sub-block 2c, their high nibbles those of sub-block 2c+1 (one AND per four
// weights, no permutation: the activations keep their natural order).  The
// output lane of weight row n is the lane that loaded row n's header, so
// d*sc_j and dmin are applied in place:
//   y[col] += d*sc_j * (dx_j[col] * idot)      per sub-block, 12 vector ops for 4 columns
//   y[col] -= dmin * sum_j m_j * s_j[col]      two v_mfma_f32_16x16x4_f32
// Workgroup = 16 waves, one per CU; the waves share 16 weight rows, one
// superblock column each, and their partial sums meet in LDS in wave order.
// LDS: codes [sub-block][NCL columns][32 B] (a wave's A read is 512 contiguous
// bytes), d and s as [sub-block][NCL] floats.
// ---------------------------------------------------------------------------
constexpr uint32_t kQ8MfmaMinCols = 4;   // measured on 12288x4096: the dot4 kernel wins up to 3 columns (12.2 against 14.9 us at 2, 16.6 against 15.1 at 4)
constexpr int kMThreads = 1024;
constexpr int kMWaves = kMThreads / LEV_WAVE;
typedef int lev_i32x4 __attribute__((ext_vector_type(4)));
constexpr int kQ8mPieces = 6;   // 16-byte pieces of a column's codes a thread stages without a loop

struct q8m_regs {
    lev_u32x4 hdr, a, b;
};

// Three 16-byte loads per lane: the header, and bytes [16*(g/2), +16) of chunk
// 2i + g%2 for i = 0, 1: a wave's load covers 64 contiguous bytes per row (five
// loads of 8 bytes cost more in the L1 than the bytes they save).
__device__ __forceinline__ void q8m_issue(const uint8_t *__restrict__ w, uint64_t row_bytes, uint32_t row,
                                          uint32_t sb, uint32_t g, q8m_regs &R) {
    const uint8_t *p = w + (uint64_t)row * row_bytes + (uint64_t)sb * 144u;
    R.hdr = *reinterpret_cast<const lev_u32x4 *>(p);
    const uint8_t *q = p + 16u + 32u * (g & 1u) + 16u * (g >> 1);
    R.a = *reinterpret_cast<const lev_u32x4 *>(q);
    R.b = *reinterpret_cast<const lev_u32x4 *>(q + 64u);
}

// The MFMA wants bytes [8g, 8g+8) of every chunk in lane group g.  Lane groups g
// and g^1 (16 lanes apart) hold each other's second piece; one row swap per dword
// puts both in place: afterwards (x, y) is the lane's piece of chunk 2i and (z, w)
// of chunk 2i+1.
__device__ __forceinline__ void q8m_exchange(lev_u32x4 &v) {
    const auto s0 = __builtin_amdgcn_permlane16_swap(v.x, v.z, false, false);
    const auto s1 = __builtin_amdgcn_permlane16_swap(v.y, v.w, false, false);
    v.x = s0[0];
    v.z = s0[1];
    v.y = s1[0];
    v.w = s1[1];
}

// NCL: columns the LDS layout holds (>= ncol).  SHORT: no wave has more than
// three tasks and a column's codes fit the unrolled staging; the kernel is then
// straight-line code (no loop holds a load), so every wait covers exactly the
// loads it needs and the first task is multiplied while the others stream in.
template <int NCL, bool SHORT>
__global__ void __launch_bounds__(kMThreads)
q4_k_q8_mfma(const uint8_t *__restrict__ w, const uint8_t *__restrict__ xq, const float *__restrict__ xs,
             float *__restrict__ y, uint32_t cols, uint32_t rows, uint32_t ncol, uint32_t lognp) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const uint32_t SB = cols >> 8, subs = cols >> 5;
    uint8_t *xa = smem;                                                  // [subs][NCL][32]
    float *sd = reinterpret_cast<float *>(smem + (size_t)cols * NCL);    // [subs][NCL]
    float *ssum = sd + (size_t)subs * NCL;                               // [subs][NCL]
    float *part = ssum + (size_t)subs * NCL;                             // [2][wave][row][NCL]

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t r = lane & 15u, g = lane >> 4;

    // ---- activations: 16 >> lognp waves per column, 16-byte pieces ----
    const uint32_t np = 1u << lognp;
    const uint32_t ac = wave & (np - 1u), apart = wave >> lognp, astride = 64u * (kMWaves >> lognp);
    const bool acol = ac < ncol;
    const uint32_t P = cols >> 4;                 // pieces per column
    const lev_u32x4 *xsrc = reinterpret_cast<const lev_u32x4 *>(xq + (uint64_t)(acol ? ac : 0u) * cols);
    const lev_u32x2 *ssrc = reinterpret_cast<const lev_u32x2 *>(xs) + (uint64_t)(acol ? ac : 0u) * subs;
    constexpr int CHX = kQ8mPieces, CHS = kQ8mPieces / 2;
    lev_u32x4 xv[CHX];
    lev_u32x2 sv[CHS];
    const uint32_t p0 = apart * 64u + lane;
#pragma unroll
    for (int i = 0; i < CHX; ++i) {
        const uint32_t p = p0 + (uint32_t)i * astride;
        xv[i] = xsrc[p < P ? p : 0u];
    }
#pragma unroll
    for (int i = 0; i < CHS; ++i) {
        const uint32_t k = p0 + (uint32_t)i * astride;
        sv[i] = ssrc[k < subs ? k : 0u];
    }

    // ---- geometry of the weight stream: task = superblock wave + 16*t of the
    // 16 rows of group rg (stride gridDim.x); a cursor walks them, no divisions.
    // A task past the end reads the first bytes of the matrix. ----
    const uint64_t row_bytes = (uint64_t)SB * 144u;
    const uint32_t ngroups = (rows + 15u) >> 4;
    const uint32_t tpr = (SB + kMWaves - 1u) / kMWaves;
    const uint32_t ntasks = ((ngroups - blockIdx.x + gridDim.x - 1u) / gridDim.x) * tpr;
    struct cursor {
        uint32_t k, rg, t;
    };
    auto advance = [&](cursor &c) {
        ++c.k;
        if (++c.t == tpr) {
            c.t = 0;
            c.rg += gridDim.x;
        }
    };
    auto issue = [&](cursor &c, q8m_regs &W) {
        const uint32_t sbw = wave + kMWaves * c.t;
        const bool real = c.k < ntasks && sbw < SB;
        uint32_t row = c.rg * 16u + r;
        row = row < rows ? row : rows - 1u;
        q8m_issue(w, row_bytes, real ? row : 0u, real ? sbw : 0u, real ? g : 0u, W);
        advance(c);
    };
    cursor ci{0u, blockIdx.x, 0u}, cc{0u, blockIdx.x, 0u};
    q8m_regs W0, W1, W2;
    issue(ci, W0);
    if constexpr (!SHORT) {
        issue(ci, W1);
        issue(ci, W2);
    }

    // the activation loads were issued first and return first
#pragma unroll
    for (int i = 0; i < CHX; ++i) {
        const uint32_t p = p0 + (uint32_t)i * astride;
        if (acol && p < P) *reinterpret_cast<lev_u32x4 *>(xa + ((size_t)(p >> 1) * NCL + ac) * 32u + (p & 1u) * 16u) = xv[i];
    }
#pragma unroll
    for (int i = 0; i < CHS; ++i) {
        const uint32_t k = p0 + (uint32_t)i * astride;
        if (acol && k < subs) {
            sd[(size_t)k * NCL + ac] = __uint_as_float(sv[i].x);
            ssum[(size_t)k * NCL + ac] = __uint_as_float(sv[i].y);
        }
    }
    if constexpr (!SHORT) if (acol) {   // columns longer than the unrolled part
        for (uint32_t p = p0 + CHX * astride; p < P; p += astride)
            *reinterpret_cast<lev_u32x4 *>(xa + ((size_t)(p >> 1) * NCL + ac) * 32u + (p & 1u) * 16u) = xsrc[p];
        for (uint32_t k = p0 + CHS * astride; k < subs; k += astride) {
            const lev_u32x2 v = ssrc[k];
            sd[(size_t)k * NCL + ac] = __uint_as_float(v.x);
            ssum[(size_t)k * NCL + ac] = __uint_as_float(v.y);
        }
    }
    lev_barrier_lds();

    // ---- stream the weights ----
    const uint32_t colc = r < (uint32_t)NCL ? r : (uint32_t)NCL - 1u;    // A rows past NCL: any valid address
    const uint32_t gq = 4u * g < (uint32_t)NCL ? 4u * g : 0u;            // first of the lane's four output columns
    const uint32_t gm8 = 8u * g;
    lev_f32x4 yacc = {0.f, 0.f, 0.f, 0.f};
    uint32_t parity = 0;
    auto compute = [&](cursor &c, const q8m_regs &W) {
        const uint32_t rg = c.rg, t = c.t;
        const uint32_t sbw = wave + kMWaves * t;
        const bool live = sbw < SB;
        const uint32_t sb = live ? sbw : SB - 1u;
        const uint32_t S0 = W.hdr.y, S1 = W.hdr.z, S2 = W.hdr.w;
        const float d = live ? lev_f16_bits_to_f32(W.hdr.x & 0xFFFFu) : 0.f;
        const float dmin = live ? lev_f16_bits_to_f32(W.hdr.x >> 16) : 0.f;
        lev_u32x4 ca = W.a, cb = W.b;
        q8m_exchange(ca);
        q8m_exchange(cb);
        const lev_u32x2 chunk[4] = {lev_u32x2{ca.x, ca.y}, lev_u32x2{ca.z, ca.w}, lev_u32x2{cb.x, cb.y},
                                    lev_u32x2{cb.z, cb.w}};
        const uint8_t *xrow = xa + ((size_t)sb * 8u * NCL + colc) * 32u + gm8;
        const float *drow = sd + (size_t)sb * 8u * NCL + gq;
        lev_f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            // unpack_scale_min, lev-cpu/src/lib.rs:64-74
            const uint32_t sc = j < 4 ? (S0 >> (8 * j)) & 63u
                                      : ((S2 >> (8 * (j - 4))) & 0xFu) | (((S0 >> (8 * (j - 4) + 6)) & 3u) << 4);
            const float scl = d * (float)sc;
            lev_u32x2 wv = chunk[j >> 1];
            if (j & 1) wv >>= 4;
            wv &= 0x0F0F0F0Fu;
            const long B = __builtin_bit_cast(long, wv);
            const long A = *reinterpret_cast<const long *>(xrow + (size_t)j * NCL * 32u);
            const lev_i32x4 D = __builtin_amdgcn_mfma_i32_16x16x32_i8(A, B, lev_i32x4{0, 0, 0, 0}, 0, 0, 0);
            const lev_f32x4 dx = *reinterpret_cast<const lev_f32x4 *>(drow + (size_t)j * NCL);
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[i] = fmaf(scl, dx[i] * (float)D[i], acc[i]);
        }
        // mins: two 16x16x4 f32 products, k = lane group: m_g and m_{4+g} of the lane's row
        const float mA = (float)((S1 >> gm8) & 63u);
        const float mB = (float)(((S2 >> (gm8 + 4u)) & 0xFu) | (((S1 >> (gm8 + 6u)) & 3u) << 4));
        const float sA = ssum[((size_t)sb * 8u + g) * NCL + colc];
        const float sB = ssum[((size_t)sb * 8u + 4u + g) * NCL + colc];
        lev_f32x4 acc2 = {0.f, 0.f, 0.f, 0.f};
        acc2 = __builtin_amdgcn_mfma_f32_16x16x4f32(sA, mA, acc2, 0, 0, 0);
        acc2 = __builtin_amdgcn_mfma_f32_16x16x4f32(sB, mB, acc2, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < 4; ++i) yacc[i] += fmaf(-dmin, acc2[i], acc[i]);

        if (t + 1u == tpr) {   // workgroup-uniform
            float *pp = part + parity * (kMWaves * 16 * NCL);   // two buffers: one barrier per group
            parity ^= 1u;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (4u * g + (uint32_t)i < (uint32_t)NCL) pp[(wave * 16u + r) * NCL + 4u * g + i] = yacc[i];
            yacc = lev_f32x4{0.f, 0.f, 0.f, 0.f};
            lev_barrier_lds();
            if (tid < 16u * NCL) {
                const uint32_t col = tid >> 4, rr = tid & 15u, row = rg * 16u + rr;
                float sum = 0.f;
#pragma unroll
                for (int kk = 0; kk < kMWaves; ++kk) sum += pp[((uint32_t)kk * 16u + rr) * NCL + col];
                if (col < ncol && row < rows) y[(uint64_t)col * rows + row] = sum;
            }
        }
        advance(c);
    };

    if constexpr (SHORT) {
        // A wave that issues a load while the CU's memory queue is full waits in the
        // issue: the second and third task are requested just ahead of the multiply
        // that precedes their use, not up front.
        issue(ci, W1);
        __builtin_amdgcn_sched_barrier(0);
        compute(cc, W0);
        __builtin_amdgcn_sched_barrier(0);
        issue(ci, W2);
        __builtin_amdgcn_sched_barrier(0);
        if (ntasks > 1u) compute(cc, W1);
        if (ntasks > 2u) compute(cc, W2);
        return;
    }
    // The scheduling barriers keep a refill's loads behind the compute that
    // frees its registers.
    while (true) {
        compute(cc, W0);
        __builtin_amdgcn_sched_barrier(0);
        issue(ci, W0);
        __builtin_amdgcn_sched_barrier(0);
        if (cc.k >= ntasks) break;
        compute(cc, W1);
        __builtin_amdgcn_sched_barrier(0);
        issue(ci, W1);
        __builtin_amdgcn_sched_barrier(0);
        if (cc.k >= ntasks) break;
        compute(cc, W2);
        __builtin_amdgcn_sched_barrier(0);
        issue(ci, W2);
        __builtin_amdgcn_sched_barrier(0);
        if (cc.k >= ntasks) break;
    }
}

// ---------------------------------------------------------------------------
// Up to four columns, rows of at most sixteen superblocks, in the shape of the f32 one-column
// kernel (q4_k_mfma_gemv_one.hip): a wave owns ONE superblock column of the matrix.  Lane (r, g)
// multiplies chunk g (32 code bytes: low nibbles = sub-block 2g, high = 2g+1) of row r by four
// v_mfma_i32_16x16x64_i8; A row 4g + c holds the 16 activation codes of column c (of a chunk of
// four columns) that lane group g multiplies, zeros elsewhere, so the four accumulator registers
// of a lane are the exact sums q * xq of its own sub-block for four columns.  The A operands are
// the activation codes as they lie in memory, so a lane loads them straight into registers, with
// the scales and sums of its two blocks beside them: nothing is staged in LDS, no barrier stands
// in front of the products.  The wave walks the row groups with the next group's weights in
// flight; the partial sums of a row meet in LDS behind one barrier per round.
// Weights: lane 4*row + c fetches dword c of the superblock's header and the 32 aligned bytes of
// chunk c (a quad reads the row's 144 contiguous bytes); one lane permutation per dword hands them
// to lane (row, c).
// LDS: part [2][16 waves][16 rows][NC] f32.
// ---------------------------------------------------------------------------
__host__ __device__ constexpr uint32_t q8m_one_part_bytes(uint32_t nc) { return 2u * kMWaves * 16u * 4u * nc; }

// NC: columns staged (a multiple of 4, >= ncol; 4 is what is built).
template <int NC>
__global__ void __launch_bounds__(kMThreads)
q4_k_q8_mfma_one(const uint8_t *__restrict__ w, const uint8_t *__restrict__ xq, const float *__restrict__ xs,
                 float *__restrict__ y, uint32_t cols, uint32_t rows, uint32_t ncol, uint32_t wpr, uint32_t slots,
                 uint64_t slot_of_wave, uint64_t pos_of_wave) {
    constexpr int NCH = NC / 4;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const uint32_t slot = (uint32_t)(slot_of_wave >> (4u * wave)) & 15u;   // idle waves: slot >= slots
    const uint32_t sb = (uint32_t)(pos_of_wave >> (4u * wave)) & 15u;      // the wave's superblock column
    const uint32_t SB = cols >> 8, nblk = cols >> 5;
    const uint32_t r = lane & 15u, g = lane >> 4;
    const bool active = slot < slots;

    // The first row group's weights are requested first: they come from HBM, the activations
    // (L2 hits) queue behind them and are back long before.
    const uint64_t row_bytes = (uint64_t)SB * 144u;
    const uint32_t ngroups = (rows + 15u) >> 4;
    const uint32_t nrounds = (ngroups + slots - 1u) / slots;     // rounds of `slots` row groups
    const uint32_t lrow = lane >> 2, lc = lane & 3u;             // fetch order: lane = 4 * row + chunk
    auto issue = [&](uint32_t round_block, uint32_t (&D)[9]) {
        uint32_t rg = round_block * slots + (active ? slot : 0u);
        rg = rg < ngroups ? rg : ngroups - 1u;
        uint32_t row = rg * 16u + lrow;
        row = row < rows ? row : rows - 1u;
        const uint8_t *p = w + (uint64_t)row * row_bytes + (uint64_t)sb * 144u;
        D[0] = *reinterpret_cast<const uint32_t *>(p + 4u * lc);
        const lev_u32x4 a = *reinterpret_cast<const lev_u32x4 *>(p + 16u + 32u * lc);
        const lev_u32x4 b = *reinterpret_cast<const lev_u32x4 *>(p + 32u + 32u * lc);
        D[1] = a.x; D[2] = a.y; D[3] = a.z; D[4] = a.w;
        D[5] = b.x; D[6] = b.y; D[7] = b.z; D[8] = b.w;
    };
    uint32_t D[9];
    uint32_t rb = blockIdx.x;
    issue(rb, D);
    __builtin_amdgcn_sched_barrier(0);

    // the wave's activations: lane (r, g) feeds A row r = 4*gs + c, i.e. column 4*ch + r%4, the 16
    // codes 64g + 16h .. of the superblock (h = 0, 1: sub-block 2g; 2, 3: sub-block 2g+1), when
    // gs == g, zeros otherwise (columns beyond ncol repeat the last one: their scales are zeroed)
    lev_i32x4 A[NCH][4];
    float dxa[NCH][4], dxb[NCH][4], sa[NCH][4], sbm[NCH][4];     // scale and sum of blocks 2g and 2g+1, column 4*ch + i
#pragma unroll
    for (int ch = 0; ch < NCH; ++ch) {
        const uint32_t ca = 4u * (uint32_t)ch + (r & 3u);
        const uint8_t *xa = xq + (uint64_t)(ca < ncol ? ca : ncol - 1u) * cols + 256u * sb + 64u * g;
#pragma unroll
        for (int h = 0; h < 4; ++h) A[ch][h] = *reinterpret_cast<const lev_i32x4 *>(xa + 16 * h);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t ci = 4u * (uint32_t)ch + (uint32_t)i;
            const lev_f32x4 t = *reinterpret_cast<const lev_f32x4 *>(
                xs + ((uint64_t)(ci < ncol ? ci : ncol - 1u) * nblk + 8u * sb + 2u * g) * 2u);
            const bool on = active && ci < ncol;
            dxa[ch][i] = on ? t.x : 0.f;
            sa[ch][i] = on ? t.y : 0.f;
            dxb[ch][i] = on ? t.z : 0.f;
            sbm[ch][i] = on ? t.w : 0.f;
        }
    }

    // ---- everything the tail of a round needs, while the loads are on their way ----
    // byte offsets into the workgroup's LDS, not pointers
    uint32_t pw = ((wave * 16u + r) * NC + g) * 4u;              // lane (r, g): row r, column g (+ 4 per chunk)
    uint32_t pr = ((((wave < slots ? wave : 0u) * wpr) * 16u + r) * NC + g) * 4u;
    uint32_t orow = (rb * slots + wave) * 16u + r;
    const uint32_t orow_step = gridDim.x * slots * 16u;
    const bool writer = wave < slots;
    uint32_t stores = writer && orow < rows ? 1u : 0u;
    uint64_t yp = reinterpret_cast<uint64_t>(y + (uint64_t)g * rows + orow);
    lev_pin(pw);
    lev_pin(pr);
    lev_pin(stores);
    lev_pin(yp);
    {
        const bool feeds = active && (r >> 2) == g;
#pragma unroll
        for (int ch = 0; ch < NCH; ++ch)
#pragma unroll
            for (int h = 0; h < 4; ++h) A[ch][h] = feeds ? A[ch][h] : lev_i32x4{0, 0, 0, 0};
    }
    __builtin_amdgcn_sched_barrier(0);

    // A round: the fetched dwords go to the lanes that multiply them, and the registers they came
    // in take the NEXT round's request at once (unconditional, clamped: a branch around the loads
    // would make the compiler wait for them before the current group is multiplied).
    auto round = [&](uint32_t next_block) {
        // lane (r, g) <- lane 4r + g for the chunk, lanes 4r .. 4r + 3 for the header's four dwords
        uint32_t hdr[4];
        lev_u32x4 ca, cb;
#pragma unroll
        for (int k = 0; k < 4; ++k) hdr[k] = (uint32_t)__builtin_amdgcn_ds_bpermute((int)(16u * r + 4u * k), (int)D[0]);
        const int src = (int)((4u * r + g) * 4u);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            ca[k] = (uint32_t)__builtin_amdgcn_ds_bpermute(src, (int)D[1 + k]);
            cb[k] = (uint32_t)__builtin_amdgcn_ds_bpermute(src, (int)D[5 + k]);
        }
        __builtin_amdgcn_sched_barrier(0);
        issue(next_block, D);
        __builtin_amdgcn_sched_barrier(0);
        // unpack_scale_min (lev-cpu/src/lib.rs:64-74), four sub-blocks a word; this lane wants sub-blocks
        // 2g and 2g + 1: bytes 2 * (g % 2) and + 1 of word g / 2 (both words are formed and one is
        // kept by a bit select: a conditional here becomes a branch)
        const uint32_t S0 = hdr[1], S1 = hdr[2], S2 = hdr[3];
        const uint32_t up = g >= 2u ? ~0u : 0u;
        const uint32_t sc_hi = (S2 & 0x0F0F0F0Fu) | ((S0 >> 2) & 0x30303030u), sc_lo = S0 & 0x3F3F3F3Fu;
        const uint32_t mn_hi = ((S2 >> 4) & 0x0F0F0F0Fu) | ((S1 >> 2) & 0x30303030u), mn_lo = S1 & 0x3F3F3F3Fu;
        const uint32_t scw = (sc_hi & up) | (sc_lo & ~up);
        const uint32_t mnw = (mn_hi & up) | (mn_lo & ~up);
        const uint32_t sh = 16u * (g & 1u);
        const float d = lev_f16_bits_to_f32(hdr[0] & 0xFFFFu);
        const float dmin = lev_f16_bits_to_f32(hdr[0] >> 16);
        const float sca = d * (float)__builtin_amdgcn_ubfe(scw, sh, 8u);
        const float scb = d * (float)__builtin_amdgcn_ubfe(scw, sh + 8u, 8u);
        const float mna = dmin * (float)__builtin_amdgcn_ubfe(mnw, sh, 8u);
        const float mnb = dmin * (float)__builtin_amdgcn_ubfe(mnw, sh + 8u, 8u);
        const lev_i32x4 la = __builtin_bit_cast(lev_i32x4, ca & 0x0F0F0F0Fu);
        const lev_i32x4 lb = __builtin_bit_cast(lev_i32x4, cb & 0x0F0F0F0Fu);
        const lev_i32x4 ha = __builtin_bit_cast(lev_i32x4, (ca >> 4) & 0x0F0F0F0Fu);
        const lev_i32x4 hb = __builtin_bit_cast(lev_i32x4, (cb >> 4) & 0x0F0F0F0Fu);
#pragma unroll
        for (int ch = 0; ch < NCH; ++ch) {
            lev_i32x4 d0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[ch][0], la, lev_i32x4{0, 0, 0, 0}, 0, 0, 0);
            lev_i32x4 d1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[ch][2], ha, lev_i32x4{0, 0, 0, 0}, 0, 0, 0);
            d0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[ch][1], lb, d0, 0, 0, 0);
            d1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[ch][3], hb, d1, 0, 0, 0);
            float v[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                // y += d*sc_j*dx_j*idot - dmin*m_j*s_j for the lane's two sub-blocks
                float t = fmaf(sca, dxa[ch][i] * (float)d0[i], -mna * sa[ch][i]);
                t = fmaf(scb, dxb[ch][i] * (float)d1[i], t);
                v[i] = fmaf(-mnb, sbm[ch][i], t);
            }
            // the four lane groups' shares of a row meet, lane group g keeping column 4*ch + g
            *reinterpret_cast<float *>(smem + pw + 16 * ch) = lev_lanegroup_sums4(v);
        }
        lev_barrier_lds();
        if (wave < slots) {
            const float *pp = reinterpret_cast<const float *>(smem + pr);
#pragma unroll
            for (int ch = 0; ch < NCH; ++ch) {
                // the slot's waves in order, four chains added at the end (sixteen reads in flight)
                float s4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int k = 0; k < kMWaves; ++k) {
                    const float pk = pp[k * 16 * NC + 4 * ch];
                    s4[k & 3] += (uint32_t)k < wpr ? pk : 0.f;
                }
                const float s = (s4[0] + s4[1]) + (s4[2] + s4[3]);
                if (stores && 4u * (uint32_t)ch + g < ncol)
                    *reinterpret_cast<__attribute__((address_space(1))) float *>(yp + (uint64_t)(4 * ch) * rows * 4u) = s;
            }
        }
        pw ^= kMWaves * 16u * 4u * NC;                          // the other half of `part` next round
        pr ^= kMWaves * 16u * 4u * NC;
        orow += orow_step;
        yp += (uint64_t)orow_step * 4u;
        stores = writer && orow < rows ? 1u : 0u;
    };
    while (true) {
        const uint32_t next = rb + gridDim.x;
        round(next < nrounds ? next : rb);
        if (next >= nrounds) break;
        rb = next;
    }
}

template <int NC>
hipError_t launch_q8m_one(lev_ctx *ctx, const uint8_t *w, const uint8_t *xq, const float *xs, float *y,
                          uint32_t cols, uint32_t rows, uint32_t ncol) {
    const uint32_t wpr = cols >> 8, slots = (uint32_t)kMWaves / wpr;
    const uint32_t ngroups = (rows + 15u) / 16u;
    const uint32_t nrounds = (ngroups + slots - 1u) / slots;
    uint64_t slot_of_wave, pos_of_wave;
    lev_wave_tables(wpr, &slot_of_wave, &pos_of_wave);
    const uint32_t blocks = nrounds < (uint32_t)ctx->num_cus ? nrounds : (uint32_t)ctx->num_cus;
    static_assert(q8m_one_part_bytes(NC) <= 48u * 1024u, "fits the default dynamic LDS limit");
    hipLaunchKernelGGL((q4_k_q8_mfma_one<NC>), dim3(blocks), dim3(kMThreads), q8m_one_part_bytes(NC), ctx->stream, w,
                       xq, xs, y, cols, rows, ncol, wpr, slots, slot_of_wave, pos_of_wave);
    return hipGetLastError();
}

size_t q8m_lds_bytes(uint32_t cols, uint32_t ncl) {
    return (size_t)cols * ncl + (size_t)2 * (cols >> 5) * ncl * 4 + (size_t)2 * kMWaves * 16 * ncl * 4;
}

template <int NCL, bool SHORT>
hipError_t launch_q8m_variant(lev_ctx *ctx, const uint8_t *w, const uint8_t *xq, const float *xs, float *y,
                              uint32_t cols, uint32_t rows, uint32_t ncol, uint32_t blocks) {
    const size_t lds = q8m_lds_bytes(cols, NCL);
    static size_t configured = 0;   // per instantiation: raise the dynamic LDS limit once per size
    if (lds > 48 * 1024 && lds > configured) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&q4_k_q8_mfma<NCL, SHORT>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        configured = lds;
    }
    uint32_t lognp = 0;
    while ((1u << lognp) < ncol) ++lognp;
    hipLaunchKernelGGL((q4_k_q8_mfma<NCL, SHORT>), dim3(blocks), dim3(kMThreads), lds, ctx->stream, w, xq,
                       xs, y, cols, rows, ncol, lognp);
    return hipGetLastError();
}

template <int NCL>
hipError_t launch_q8m(lev_ctx *ctx, const uint8_t *w, const uint8_t *xq, const float *xs, float *y,
                      uint32_t cols, uint32_t rows, uint32_t ncol) {
    const uint32_t groups = (rows + 15u) / 16u;
    const uint32_t blocks = groups < (uint32_t)ctx->num_cus ? groups : (uint32_t)ctx->num_cus;
    const uint32_t tpr = ((cols >> 8) + kMWaves - 1u) / kMWaves;
    const uint32_t most = ((groups + blocks - 1u) / blocks) * tpr;   // tasks of the busiest wave
    uint32_t lognp = 0;
    while ((1u << lognp) < ncol) ++lognp;
    const bool staged = (cols >> 4) <= kQ8mPieces * 64u * ((uint32_t)kMWaves >> lognp);
    if (most <= 3u && staged)
        return launch_q8m_variant<NCL, true>(ctx, w, xq, xs, y, cols, rows, ncol, blocks);
    return launch_q8m_variant<NCL, false>(ctx, w, xq, xs, y, cols, rows, ncol, blocks);
}

// Columns one launch of the matrix-core kernel takes for this in_dim (0: none).
uint32_t q8m_cols(const lev_ctx *ctx, uint32_t in_dim) {
    const size_t limit = ctx->props.sharedMemPerBlockOptin > ctx->props.sharedMemPerBlock
                             ? ctx->props.sharedMemPerBlockOptin
                             : ctx->props.sharedMemPerBlock;
    for (uint32_t ncl = 16; ncl >= 4u; ncl >>= 1)
        if (q8m_lds_bytes(in_dim, ncl) <= limit) return ncl;
    return 0;
}

}  // namespace

extern "C" int lev_hip_norm_quant_q8(lev_ctx *ctx, float *d_x, size_t x_count, const float *d_add,
                                     const float *d_gain, float eps, int8_t *d_xq, float *d_xs,
                                     float *d_y, uint32_t n, uint32_t ncol) {
    LEV_REQUIRE_CTX(ctx);
    if (!d_x || !d_xq || !d_xs) return lev_fail(ctx, LEV_ERR_INVALID_ARGUMENT, "norm_quant_q8: null pointer");
    if (n == 0 || n % 32u != 0u || n > LEV_MAX_Q4_INPUT_DIM || ncol == 0 || ncol > 65535u)
        return lev_fail(ctx, LEV_ERR_BAD_DIMENSIONS, "norm_quant_q8: n %u (multiple of 32), %u columns", n, ncol);
    if (x_count != (size_t)n * ncol)
        return lev_fail(ctx, LEV_ERR_WRONG_INPUT_COUNT, "norm_quant_q8: %zu activations, need %zu", x_count,
                        (size_t)n * ncol);
    if (d_gain && !(eps >= 0.f)) return lev_fail(ctx, LEV_ERR_BAD_DIMENSIONS, "norm_quant_q8: eps %g", (double)eps);
    if ((reinterpret_cast<uintptr_t>(d_xq) & 3u) || (reinterpret_cast<uintptr_t>(d_xs) & 7u))
        return lev_fail(ctx, LEV_ERR_BAD_DIMENSIONS, "norm_quant_q8: xq must be 4-byte, xs 8-byte aligned");
    if ((reinterpret_cast<uintptr_t>(d_x) | reinterpret_cast<uintptr_t>(d_add) |
         reinterpret_cast<uintptr_t>(d_gain) | reinterpret_cast<uintptr_t>(d_y)) & 15u)
        return lev_fail(ctx, LEV_ERR_BAD_DIMENSIONS, "norm_quant_q8: x, add, gain and y must be 16-byte aligned");
    hipLaunchKernelGGL(norm_quant_kernel, dim3(ncol), dim3(kNQThreads), 0, ctx->stream, d_x, d_add, d_gain,
                       eps, reinterpret_cast<uint32_t *>(d_xq), d_xs, d_y, n);
    return lev_hip_check(ctx, hipGetLastError(), "norm_quant_q8 launch");
}

// Candidate schedules of a Q4_K x int8 GEMV shape, the built-in choice first:
// the dot4 kernel and, where its staging fits, the integer matrix-core kernel.
uint32_t lev_q4_k_gemv_q8_candidates(const lev_ctx *ctx, uint32_t in_dim, uint32_t rows, uint32_t ncol,
                                     lev_schedule *out, uint32_t capacity) {
    (void)rows;
    const bool has_mfma = q8m_cols(ctx, in_dim) != 0u;
    // built-in: the matrix cores for every column count of rows up to 4096 wide (a wave per
    // superblock column up to four columns), from kQ8MfmaMinCols columns for wider rows
    const uint32_t first = has_mfma && (ncol >= kQ8MfmaMinCols || in_dim <= 4096u) ? 1u : 0u;
    uint32_t n = 0;
    if (n < capacity) out[n] = lev_schedule{LEV_OP_Q4_K_GEMV_Q8, first, 0u, 0u};
    ++n;
    if (has_mfma) {
        if (n < capacity) out[n] = lev_schedule{LEV_OP_Q4_K_GEMV_Q8, 1u - first, 0u, 0u};
        ++n;
    }
    return n;
}

extern "C" int lev_hip_q4_k_gemv_q8(lev_ctx *ctx, const void *d_w, size_t w_bytes, uint64_t w_off,
                                    const int8_t *d_xq, const float *d_xs, size_t x_count, float *d_y,
                                    size_t y_capacity, uint32_t in_dim, uint32_t rows, uint32_t ncol) {
    LEV_REQUIRE_CTX(ctx);
    if (ncol == 0 || ncol > LEV_MAX_GEMV_COLUMNS)
        return lev_fail(ctx, LEV_ERR_BAD_DIMENSIONS, "q4_k_gemv_q8: %u columns (1..%d)", ncol,
                        LEV_MAX_GEMV_COLUMNS);
    if (!d_xs) return lev_fail(ctx, LEV_ERR_INVALID_ARGUMENT, "q4_k_gemv_q8: null pointer");
    lev_geom g;
    int st = lev_check_matvec(ctx, "q4_k_gemv_q8", 256, 144, d_w, w_bytes, w_off, d_xq, x_count,
                              (uint64_t)in_dim * ncol, d_y, y_capacity, (uint64_t)rows * ncol, in_dim, rows,
                              &g);
    if (st != LEV_OK) return st;
    const uint8_t *w = static_cast<const uint8_t *>(d_w) + w_off;
    if ((reinterpret_cast<uintptr_t>(w) & 15u) || (reinterpret_cast<uintptr_t>(d_xq) & 15u) ||
        (reinterpret_cast<uintptr_t>(d_xs) & 15u))
        return lev_fail(ctx, LEV_ERR_BAD_DIMENSIONS, "q4_k_gemv_q8: weights, xq and xs must be 16-byte aligned");
    const size_t limit = ctx->props.sharedMemPerBlockOptin > ctx->props.sharedMemPerBlock
                             ? ctx->props.sharedMemPerBlockOptin
                             : ctx->props.sharedMemPerBlock;
    const uint32_t *xq = reinterpret_cast<const uint32_t *>(d_xq);
    // Built-in choice: the matrix-core kernel from kQ8MfmaMinCols columns up, the
    // dot4 kernel below; a schedule installed for the shape (lev_hip_forge_select)
    // overrides it.
    const uint32_t mcols = q8m_cols(ctx, in_dim);
    const lev_schedule *sel = lev_selected(ctx, LEV_OP_Q4_K_GEMV_Q8, in_dim, rows, ncol);
    const bool mfma = mcols != 0u && (sel ? sel->family == 1u : (ncol >= kQ8MfmaMinCols || in_dim <= 4096u));
    // rows of at most sixteen superblocks: the matrix-core kernel with a wave per superblock column,
    // for every column count (a schedule of family 0 still selects the dot4 kernel)
    static const bool one_off = [] {
        const char *e = getenv("LEV_Q4K_Q8_ONE");   // LEV_Q4K_Q8_ONE=0: the kernels below, for comparison
        return e && e[0] == '0';
    }();
    const bool mfma_one = !one_off && in_dim <= 4096u && mfma;
    uint32_t done = 0;
    while (done < ncol) {
        uint32_t nc = ncol - done;
        const uint32_t *xqc = xq + ((uint64_t)done * in_dim >> 2);
        const float *xsc = d_xs + (uint64_t)done * (in_dim >> 5) * 2u;
        float *yc = d_y + (uint64_t)done * rows;
        hipError_t e;
        if (mfma_one && nc <= 4u) {
            // up to four columns (eight through it measured 11.9 us at 12288 x 4096, what the
            // sixteen-column kernel below takes for eight as well)
            if (nc > 4u) nc = 4u;
            e = launch_q8m_one<4>(ctx, w, reinterpret_cast<const uint8_t *>(xqc), xsc, yc, in_dim, rows, nc);
        } else if (mfma) {
            if (nc > mcols) nc = mcols;
            const uint8_t *xb = reinterpret_cast<const uint8_t *>(xqc);
            if (mcols == 16u) e = launch_q8m<16>(ctx, w, xb, xsc, yc, in_dim, rows, nc);
            else if (mcols == 8u) e = launch_q8m<8>(ctx, w, xb, xsc, yc, in_dim, rows, nc);
            else e = launch_q8m<4>(ctx, w, xb, xsc, yc, in_dim, rows, nc);
        } else {
            // columns per launch: 8, 4, 2 or 1, within the LDS budget
            uint32_t fit = 8;
            while (fit > 1u && (size_t)fit * (in_dim >> 8) * (kCodeStride + kPairStride) > limit) fit >>= 1;
            if ((size_t)(in_dim >> 8) * (kCodeStride + kPairStride) > limit)
                return lev_fail(ctx, LEV_ERR_EXCEEDS_MODEL_WORKLOAD, "q4_k_gemv_q8: inDim %u does not fit the staging", in_dim);
            if (nc > fit) nc = fit;
            if (nc > 4) e = launch_q8<8>(ctx, w, xqc, xsc, yc, in_dim, rows, nc);
            else if (nc > 2) e = launch_q8<4>(ctx, w, xqc, xsc, yc, in_dim, rows, nc);
            else if (nc > 1) e = launch_q8<2>(ctx, w, xqc, xsc, yc, in_dim, rows, nc);
            else e = launch_q8<1>(ctx, w, xqc, xsc, yc, in_dim, rows, nc);
        }
        if (e != hipSuccess) return lev_hip_check(ctx, e, "q4_k_gemv_q8 launch");
        done += nc;
    }
    return LEV_OK;
}

// Columns one pass of the Q6_K x int8 kernel takes: the staged activations of up to
// eight columns must fit the LDS (0: not even one does).
static uint32_t q6_q8_cols_per_pass(const lev_ctx *ctx, uint32_t in_dim, uint32_t ncol) {
    const size_t limit = ctx->props.sharedMemPerBlockOptin > ctx->props.sharedMemPerBlock
                             ? ctx->props.sharedMemPerBlockOptin
                             : ctx->props.sharedMemPerBlock;
    const size_t per_col = (size_t)(in_dim >> 8) * kQ6Stride;
    if (per_col > limit) return 0;
    uint32_t fit = 8;
    while (fit > 1u && fit * per_col > limit) fit >>= 1;
    uint32_t nc = 1;
    while (nc < ncol && nc < fit) nc <<= 1;   // the kernel is built for 1, 2, 4 and 8 columns
    return nc;
}

uint32_t lev_q6_k_mfma_q8_cols(const lev_ctx *ctx, uint32_t in_dim);
hipError_t lev_q6_k_mfma_gemv_q8_launch(lev_ctx *ctx, const uint8_t *w, const uint32_t *xq, const float *xs,
                                        float *y, uint32_t in_dim, uint32_t rows, uint32_t ncol, uint32_t waves);

// Candidate schedules of a Q6_K x int8 GEMV shape, the built-in choice first
// (q6k.matvec over int8 activations, lev-forge/src/q8.rs:328-447): the integer
// matrix-core kernel (family 1; rows_in_flight = columns per pass over the weights),
// then the dot4 kernel (family 0) with a resident grid or a workgroup per row tile,
// all columns in one pass over the weights or half of them in each of two.
uint32_t lev_q6_k_gemv_q8_candidates(const lev_ctx *ctx, uint32_t in_dim, uint32_t rows, uint32_t ncol,
                                     lev_schedule *out, uint32_t capacity) {
    (void)rows;
    const uint32_t all = q6_q8_cols_per_pass(ctx, in_dim, ncol);
    const uint32_t mcols = lev_q6_k_mfma_q8_cols(ctx, in_dim);
    uint32_t n = 0;
    auto add = [&](uint32_t family, uint32_t cols, uint32_t persistent) {
        if (n < capacity) out[n] = lev_schedule{LEV_OP_Q6_K_GEMV_Q8, family, cols, persistent};
        ++n;
    };
    if (mcols) add(1u, ncol < mcols ? ncol : mcols, 1u);
    if (all == 0) return n;
    add(0u, all, 1u);
    add(0u, all, 0u);
    if (all >= 2u) add(0u, all / 2u, 1u);
    return n;
}

extern "C" int lev_hip_q6_k_gemv_q8(lev_ctx *ctx, const void *d_w, size_t w_bytes, uint64_t w_off,
                                    const int8_t *d_xq, const float *d_xs, size_t x_count, float *d_y,
                                    size_t y_capacity, uint32_t in_dim, uint32_t rows, uint32_t ncol) {
    LEV_REQUIRE_CTX(ctx);
    if (ncol == 0 || ncol > LEV_MAX_GEMV_COLUMNS)
        return lev_fail(ctx, LEV_ERR_BAD_DIMENSIONS, "q6_k_gemv_q8: %u columns (1..%d)", ncol,
                        LEV_MAX_GEMV_COLUMNS);
    if (!d_xs) return lev_fail(ctx, LEV_ERR_INVALID_ARGUMENT, "q6_k_gemv_q8: null pointer");
    lev_geom g;
    int st = lev_check_matvec(ctx, "q6_k_gemv_q8", 256, 210, d_w, w_bytes, w_off, d_xq, x_count,
                              (uint64_t)in_dim * ncol, d_y, y_capacity, (uint64_t)rows * ncol, in_dim, rows,
                              &g);
    if (st != LEV_OK) return st;
    const uint8_t *w = static_cast<const uint8_t *>(d_w) + w_off;
    if ((reinterpret_cast<uintptr_t>(w) & 1u) || (reinterpret_cast<uintptr_t>(d_xq) & 15u) ||
        (reinterpret_cast<uintptr_t>(d_xs) & 7u))
        return lev_fail(ctx, LEV_ERR_BAD_DIMENSIONS,
                        "q6_k_gemv_q8: weights must be 2-byte, xq 16-byte, xs 8-byte aligned");
    const uint32_t *xq = reinterpret_cast<const uint32_t *>(d_xq);
    // a schedule installed for this shape (lev_hip_forge_select) overrides the built-in choice
    const lev_schedule *sel = lev_selected(ctx, LEV_OP_Q6_K_GEMV_Q8, in_dim, rows, ncol);
    const uint32_t mcols = lev_q6_k_mfma_q8_cols(ctx, in_dim);
    if (mcols && (!sel || sel->family == 1u)) {
        // the integer matrix-core kernel: up to mcols columns per pass over the weights
        for (uint32_t done = 0; done < ncol; done += mcols) {
            const uint32_t nc = ncol - done < mcols ? ncol - done : mcols;
            hipError_t e = lev_q6_k_mfma_gemv_q8_launch(ctx, w, xq + ((uint64_t)done * in_dim >> 2),
                                                        d_xs + (uint64_t)done * (in_dim >> 5) * 2u,
                                                        d_y + (uint64_t)done * rows, in_dim, rows, nc, 0u);
            if (e != hipSuccess) return lev_hip_check(ctx, e, "q6_k_gemv_q8 launch");
        }
        return LEV_OK;
    }
    const size_t limit = ctx->props.sharedMemPerBlockOptin > ctx->props.sharedMemPerBlock
                             ? ctx->props.sharedMemPerBlockOptin
                             : ctx->props.sharedMemPerBlock;
    const size_t per_col = (size_t)(in_dim >> 8) * kQ6Stride;
    if (per_col > limit)
        return lev_fail(ctx, LEV_ERR_EXCEEDS_MODEL_WORKLOAD, "q6_k_gemv_q8: inDim %u does not fit the staging", in_dim);
    uint32_t fit = q6_q8_cols_per_pass(ctx, in_dim, ncol);
    bool persistent = true;
    if (sel) {
        if (sel->rows_in_flight >= 1u && sel->rows_in_flight < fit) fit = sel->rows_in_flight;
        persistent = sel->persistent != 0u;
    }
    uint32_t done = 0;
    while (done < ncol) {
        uint32_t nc = ncol - done;
        if (nc > fit) nc = fit;
        const uint32_t *xqc = xq + ((uint64_t)done * in_dim >> 2);
        const float *xsc = d_xs + (uint64_t)done * (in_dim >> 5) * 2u;
        float *yc = d_y + (uint64_t)done * rows;
        hipError_t e;
        if (nc > 4) e = launch_q6_q8<8>(ctx, w, xqc, xsc, yc, in_dim, rows, nc, persistent);
        else if (nc > 2) e = launch_q6_q8<4>(ctx, w, xqc, xsc, yc, in_dim, rows, nc, persistent);
        else if (nc > 1) e = launch_q6_q8<2>(ctx, w, xqc, xsc, yc, in_dim, rows, nc, persistent);
        else e = launch_q6_q8<1>(ctx, w, xqc, xsc, yc, in_dim, rows, nc, persistent);
        if (e != hipSuccess) return lev_hip_check(ctx, e, "q6_k_gemv_q8 launch");
        done += nc;
    }
    return LEV_OK;
}

extern "C" int lev_hip_swiglu_quant_q8(lev_ctx *ctx, const float *d_gate, const float *d_up, size_t count,
                                       int8_t *d_xq, float *d_xs, float *d_act) {
    LEV_REQUIRE_CTX(ctx);
    if (!d_gate || !d_up || !d_xq || !d_xs)
        return lev_fail(ctx, LEV_ERR_INVALID_ARGUMENT, "swiglu_quant_q8: null pointer");
    if (count == 0 || count % 32u != 0u || count > ((size_t)1 << 31))
        return lev_fail(ctx, LEV_ERR_BAD_DIMENSIONS, "swiglu_quant_q8: %zu values (a multiple of 32)", count);
    if (((reinterpret_cast<uintptr_t>(d_gate) | reinterpret_cast<uintptr_t>(d_up) |
          reinterpret_cast<uintptr_t>(d_act)) & 15u) ||
        (reinterpret_cast<uintptr_t>(d_xq) & 3u) || (reinterpret_cast<uintptr_t>(d_xs) & 7u))
        return lev_fail(ctx, LEV_ERR_BAD_DIMENSIONS,
                        "swiglu_quant_q8: gate, up and act must be 16-byte, xq 4-byte, xs 8-byte aligned");
    const uint32_t n4 = (uint32_t)(count >> 2);
    hipLaunchKernelGGL(swiglu_quant_kernel, dim3((n4 + 255u) / 256u), dim3(256), 0, ctx->stream, d_gate, d_up,
                       reinterpret_cast<uint32_t *>(d_xq), d_xs, d_act, n4);
    return lev_hip_check(ctx, hipGetLastError(), "swiglu_quant_q8 launch");
}

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
            __syncthreads();
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
constexpr int kQThreads = 256;
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
    __syncthreads();

    const uint32_t grp = lane >> 4, lp = lane & 15u;
    const uint64_t row_bytes = (uint64_t)SB * 144u;
    const uint32_t tiles = (rows + 15u) >> 4;          // 16 rows per workgroup tile
    for (uint32_t tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
        const uint32_t row = tile * 16u + wave * 4u + grp;
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
    const uint32_t tiles = (rows + 15u) / 16u;
    uint32_t blocks = (uint32_t)ctx->num_cus * (uint32_t)per_cu;
    if (blocks > tiles) blocks = tiles;
    hipLaunchKernelGGL((q4_k_gemv_q8_kernel<NC>), dim3(blocks), dim3(kQThreads), lds, ctx->stream, w, xq,
                       xs, y, in_dim, rows, ncol);
    return hipGetLastError();
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
    uint32_t done = 0;
    while (done < ncol) {
        uint32_t nc = ncol - done;
        // columns per launch: 8, 4, 2 or 1, within the LDS budget
        uint32_t fit = 8;
        while (fit > 1u && (size_t)fit * (in_dim >> 8) * (kCodeStride + kPairStride) > limit) fit >>= 1;
        if ((size_t)(in_dim >> 8) * (kCodeStride + kPairStride) > limit)
            return lev_fail(ctx, LEV_ERR_EXCEEDS_MODEL_WORKLOAD, "q4_k_gemv_q8: inDim %u does not fit the staging", in_dim);
        if (nc > fit) nc = fit;
        const uint32_t *xqc = xq + ((uint64_t)done * in_dim >> 2);
        const float *xsc = d_xs + (uint64_t)done * (in_dim >> 5) * 2u;
        float *yc = d_y + (uint64_t)done * rows;
        hipError_t e;
        if (nc > 4) e = launch_q8<8>(ctx, w, xqc, xsc, yc, in_dim, rows, nc);
        else if (nc > 2) e = launch_q8<4>(ctx, w, xqc, xsc, yc, in_dim, rows, nc);
        else if (nc > 1) e = launch_q8<2>(ctx, w, xqc, xsc, yc, in_dim, rows, nc);
        else e = launch_q8<1>(ctx, w, xqc, xsc, yc, in_dim, rows, nc);
        if (e != hipSuccess) return lev_hip_check(ctx, e, "q4_k_gemv_q8 launch");
        done += nc;
    }
    return LEV_OK;
}

// Q4_K multi-column GEMV with the RMSNorm of the input fused in front (gfx950).
//
// Stands in for Builder::norm_quant + Builder::matvec of the MTP verify step
// (rust/crates/lev-model/src/gpu.rs:295, 334-370), i.e. the GLSL q4k.matvec
// with nb columns per weight read (lev-forge/src/glsl.rs:157-281), in f32
// activations.  x is [ncol][in_dim], y is [ncol][rows].
//
// Layout in HBM is the GGUF one: 144-byte superblocks of 256 weights
// (fp16 d, fp16 dmin, 12 bytes of packed 6-bit scales/mins, 128 code bytes;
// lev-cpu/src/lib.rs:62-131), 16-byte aligned when the tensor is.
//
// Work unit: one 32-byte chunk of codes = 64 consecutive weights (low nibbles
// -> elements 0..31 with sub-block 2c, high nibbles -> 32..63 with sub-block
// 2c+1) plus the superblock's 16-byte header: three 128-bit loads per lane,
// 64 lanes cover a 4096-wide row contiguously.  Weights are decoded once per
// row and applied to every column (factored form
//   d*sc*sum(q*x) - dmin*m*sum(x)   per 32-weight sub-block).
// RMSNorm: while staging x*gain into LDS each workgroup also accumulates
// sum(x^2) per column; 1/rms is applied to the finished dot products, so the
// reduction never sits on the critical path.
#include "lev_common.hpp"

namespace {

constexpr int kThreads = 512;
constexpr int kWaves = kThreads / LEV_WAVE;

struct q4k_unit_w {
    uint32_t hdr[4];   // d | dmin<<16, scales[0..3], scales[4..7], scales[8..11]
    uint32_t qs[8];
};

__device__ __forceinline__ void q4k_load_unit(const uint8_t *row, uint32_t u, q4k_unit_w &w) {
    const uint8_t *blk = row + (uint64_t)(u >> 2) * 144u;
    lev_u32x4 h = *reinterpret_cast<const lev_u32x4 *>(blk);
    lev_u32x4 a = *reinterpret_cast<const lev_u32x4 *>(blk + 16u + 32u * (u & 3u));
    lev_u32x4 b = *reinterpret_cast<const lev_u32x4 *>(blk + 32u + 32u * (u & 3u));
    w.hdr[0] = h.x; w.hdr[1] = h.y; w.hdr[2] = h.z; w.hdr[3] = h.w;
    w.qs[0] = a.x; w.qs[1] = a.y; w.qs[2] = a.z; w.qs[3] = a.w;
    w.qs[4] = b.x; w.qs[5] = b.y; w.qs[6] = b.z; w.qs[7] = b.w;
}

// The four factors of unit chunk c (sub-blocks 2c and 2c+1):
//   f[0] = d*sc(2c) * 2^24, f[1] = d*sc(2c+1) * 2^24,
//   f[2] = dmin*m(2c),      f[3] = dmin*m(2c+1)
// (unpack_scale_min, lev-cpu/src/lib.rs:64-74).  The 2^24 undoes the fp16
// subnormal encoding of the codes.
__device__ __forceinline__ void q4k_factors(const q4k_unit_w &w, uint32_t c, float f[4]) {
    const float d = lev_f16_bits_to_f32(w.hdr[0] & 0xFFFFu);
    const float dmin = lev_f16_bits_to_f32(w.hdr[0] >> 16);
    // scale bytes as two 16-bit pairs: lo16(x) = bytes (j, j+1)
    const uint32_t sh = 16u * (c & 1u);
    const uint32_t s03 = w.hdr[1], s47 = w.hdr[2], s811 = w.hdr[3];
    uint32_t sc0, sc1, m0, m1;
    if (c < 2u) {
        uint32_t a = s03 >> sh, b = s47 >> sh;          // bytes j, j+1 and j+4, j+5
        sc0 = a & 63u;
        sc1 = (a >> 8) & 63u;
        m0 = b & 63u;
        m1 = (b >> 8) & 63u;
    } else {
        uint32_t a = s811 >> sh, lo = s03 >> sh, hi = s47 >> sh;   // bytes j+4.., j-4.., j..
        sc0 = (a & 0x0Fu) | ((lo >> 2) & 0x30u);
        sc1 = ((a >> 8) & 0x0Fu) | ((lo >> 10) & 0x30u);
        m0 = ((a >> 4) & 0x0Fu) | ((hi >> 2) & 0x30u);
        m1 = ((a >> 12) & 0x0Fu) | ((hi >> 10) & 0x30u);
    }
    const float d24 = d * 16777216.0f;
    f[0] = d24 * (float)sc0;
    f[1] = d24 * (float)sc1;
    f[2] = dmin * (float)m0;
    f[3] = dmin * (float)m1;
}

// Codes of one unit as fp16 subnormals: m[4t+0] = bytes 0,2 low nibbles,
// m[4t+1] = bytes 1,3 low, m[4t+2] = bytes 0,2 high (x16), m[4t+3] = bytes 1,3 high (x16).
__device__ __forceinline__ void q4k_mask_codes(const q4k_unit_w &w, uint32_t m[32]) {
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        uint32_t v = w.qs[t], s = v >> 8;
        m[4 * t + 0] = v & 0x000F000Fu;
        m[4 * t + 1] = s & 0x000F000Fu;
        m[4 * t + 2] = v & 0x00F000F0u;
        m[4 * t + 3] = s & 0x00F000F0u;
    }
}

struct q4k_unit_x {
    lev_f32x4 xr[16];      // xr[t] = elements 4t..4t+3 of the unit's 64
    float sum_lo, sum_hi;  // sums of elements 0..31 and 32..63
};

// sum(q*x) over the low and the high sub-block, both scaled by 2^-24.
__device__ __forceinline__ void q4k_dots(const uint32_t m[32], const q4k_unit_x &x, float &lo,
                                         float &hi) {
    float l0 = 0.f, l1 = 0.f, h0 = 0.f, h1 = 0.f;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        lev_f16x2 a = __builtin_bit_cast(lev_f16x2, m[4 * t + 0]);
        lev_f16x2 b = __builtin_bit_cast(lev_f16x2, m[4 * t + 1]);
        lev_f16x2 c = __builtin_bit_cast(lev_f16x2, m[4 * t + 2]);
        lev_f16x2 d = __builtin_bit_cast(lev_f16x2, m[4 * t + 3]);
        lev_f32x4 xl = x.xr[t], xh = x.xr[8 + t];
        l0 = fmaf((float)a.x, xl.x, l0);
        l1 = fmaf((float)b.x, xl.y, l1);
        l0 = fmaf((float)a.y, xl.z, l0);
        l1 = fmaf((float)b.y, xl.w, l1);
        h0 = fmaf((float)c.x, xh.x, h0);
        h1 = fmaf((float)d.x, xh.y, h1);
        h0 = fmaf((float)c.y, xh.z, h0);
        h1 = fmaf((float)d.y, xh.w, h1);
    }
    lo = l0 + l1;
    hi = (h0 + h1) * 0.0625f;
}

__device__ __forceinline__ float q4k_combine(const float f[4], float lo, float hi,
                                             const q4k_unit_x &x) {
    float pos = fmaf(f[0], lo, f[1] * hi);
    float neg = fmaf(f[2], x.sum_lo, f[3] * x.sum_hi);
    return pos - neg;
}

__device__ __forceinline__ void q4k_fetch_x(const lev_f32x4 *xs, uint32_t units, uint32_t u,
                                            q4k_unit_x &x) {
#pragma unroll
    for (int q = 0; q < 16; ++q) x.xr[q] = xs[q * (units + 1u) + u];
    float a = 0.f, b = 0.f;
#pragma unroll
    for (int q = 0; q < 8; ++q) {
        a += (x.xr[q].x + x.xr[q].y) + (x.xr[q].z + x.xr[q].w);
        b += (x.xr[8 + q].x + x.xr[8 + q].y) + (x.xr[8 + q].z + x.xr[8 + q].w);
    }
    x.sum_lo = a;
    x.sum_hi = b;
}

// NC columns, L lanes per row.  LDS: NC vectors in the unit-major transposed
// layout (float4 slot q*(U+1)+u of column c at c*16*(U+1)), then NC floats of
// 1/rms.  One row per wave-group and tile, persistent, double-buffered.
// One column fits in 128 registers: four waves per SIMD, i.e. four workgroups per CU.
template <int NC, int L, bool RESIDENT>
__global__ void __launch_bounds__(kThreads, (NC == 1 && RESIDENT) ? 4 : 1)
q4_k_gemv_ncol(const uint8_t *__restrict__ w, const float *__restrict__ x,
               const float *__restrict__ gain, float eps, float *__restrict__ y, uint32_t units,
               uint32_t rows) {
    extern __shared__ lev_f32x4 xs[];
    __shared__ float s_part[NC][kWaves];
    __shared__ float s_inv[NC];
    constexpr int G = LEV_WAVE / L;
    constexpr uint32_t kRowsPerTile = kWaves * G;
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & (LEV_WAVE - 1);
    const uint32_t wave = tid / LEV_WAVE;
    const uint32_t grp = lane / L, lu = lane % L;
    const uint32_t in_dim = units * 64u;
    const uint64_t row_bytes = (uint64_t)(units >> 2) * 144u;
    const uint32_t in_tile = wave * G + grp;
    const uint32_t step = gridDim.x * kRowsPerTile;
    const uint32_t col_slots = 16u * (units + 1u);

    uint32_t base = blockIdx.x * kRowsPerTile;
    if (base >= rows) return;

    // First tile's weights go out first; lanes past the end read a valid unit
    // and get zero factors.
    q4k_unit_w Wa, Wb;
    const uint32_t u0 = lu < units ? lu : units - 1u;
    {
        uint32_t row = base + in_tile;
        q4k_load_unit(w + (uint64_t)(row < rows ? row : rows - 1u) * row_bytes, u0, Wa);
    }

    // Stage x*gain and accumulate sum(x^2) per column.
    {
        const lev_f32x4 *g4 = reinterpret_cast<const lev_f32x4 *>(gain);
        const uint32_t n4 = units * 16u;
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            const lev_f32x4 *x4 = reinterpret_cast<const lev_f32x4 *>(x + (uint64_t)c * in_dim);
            float ss = 0.f;
            for (uint32_t i = tid; i < n4; i += kThreads) {
                lev_f32x4 v = x4[i];
                ss = fmaf(v.x, v.x, ss);
                ss = fmaf(v.y, v.y, ss);
                ss = fmaf(v.z, v.z, ss);
                ss = fmaf(v.w, v.w, ss);
                if (gain) {
                    lev_f32x4 g = g4[i];
                    v.x *= g.x; v.y *= g.y; v.z *= g.z; v.w *= g.w;
                }
                xs[c * col_slots + (i & 15u) * (units + 1u) + (i >> 4)] = v;
            }
            ss = lev_group_sum<64>(ss);
            if (lane == LEV_WAVE - 1) s_part[c][wave] = ss;
        }
    }
    lev_barrier_lds();
    if (tid < NC) {
        float inv = 1.0f;
        if (gain) {
            double tot = 0.0;
#pragma unroll
            for (int k = 0; k < kWaves; ++k) tot += (double)s_part[tid][k];
            inv = (float)(1.0 / sqrt(tot / (double)in_dim + (double)eps));
        }
        s_inv[tid] = inv;
    }
    lev_barrier_lds();

    q4k_unit_x X[RESIDENT ? NC : 1];
    if (RESIDENT) {
#pragma unroll
        for (int c = 0; c < NC; ++c) q4k_fetch_x(xs + c * col_slots, units, u0, X[c]);
    }
    float inv[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) inv[c] = s_inv[c];

    auto finish = [&](uint32_t row, const q4k_unit_w &W0) {
        float acc[NC];
#pragma unroll
        for (int c = 0; c < NC; ++c) acc[c] = 0.f;
        q4k_unit_w W = W0;
        const bool row_ok = row < rows;
        const uint8_t *rp = w + (uint64_t)(row_ok ? row : rows - 1u) * row_bytes;
        for (uint32_t ub = 0; ub < units; ub += L) {
            const uint32_t u = ub + lu;
            const uint32_t uc = u < units ? u : units - 1u;
            if (ub != 0) q4k_load_unit(rp, uc, W);
            float f[4];
            q4k_factors(W, uc & 3u, f);
            if (!(row_ok && u < units)) f[0] = f[1] = f[2] = f[3] = 0.f;
            uint32_t m[32];
            q4k_mask_codes(W, m);
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                float lo, hi;
                if (RESIDENT) {
                    q4k_dots(m, X[c], lo, hi);
                    acc[c] += q4k_combine(f, lo, hi, X[c]);
                } else {
                    q4k_fetch_x(xs + c * col_slots, units, uc, X[0]);
                    q4k_dots(m, X[0], lo, hi);
                    acc[c] += q4k_combine(f, lo, hi, X[0]);
                }
            }
            if (RESIDENT) break;   // resident kernels cover the row in one pass
        }
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            float s = lev_group_sum<L>(acc[c]);
            if (lu == L - 1 && row_ok) y[(uint64_t)c * rows + row] = s * inv[c];
        }
    };

    // the next tile is requested unconditionally (clamped past the end): a branch
    // around the loads would make the compiler wait for them before the current
    // tile is used
    while (true) {
        uint32_t next = base + step;
        {
            uint32_t row = next + in_tile;
            q4k_load_unit(w + (uint64_t)(row < rows ? row : rows - 1u) * row_bytes, u0, Wb);
        }
        finish(base + in_tile, Wa);
        if (next >= rows) break;
        base = next;
        next = base + step;
        {
            uint32_t row = next + in_tile;
            q4k_load_unit(w + (uint64_t)(row < rows ? row : rows - 1u) * row_bytes, u0, Wa);
        }
        finish(base + in_tile, Wb);
        if (next >= rows) break;
        base = next;
    }
}

template <int NC, int L, bool RESIDENT>
hipError_t launch_ncol(lev_ctx *ctx, const uint8_t *w, const float *x, const float *gain, float eps,
                       float *y, uint32_t units, uint32_t rows) {
    constexpr uint32_t rows_per_tile = kWaves * (LEV_WAVE / L);
    uint32_t blocks = (rows + rows_per_tile - 1) / rows_per_tile;
    size_t lds = (size_t)NC * 16 * (units + 1) * sizeof(lev_f32x4);
    if (lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(
            reinterpret_cast<const void *>(&q4_k_gemv_ncol<NC, L, RESIDENT>),
            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
    }
    // persistent grid: exactly the workgroups that are resident at once (a grid
    // larger than that runs its surplus as a second, mostly idle round)
    int resident = 0;
    hipError_t oe = hipOccupancyMaxActiveBlocksPerMultiprocessor(
        &resident, reinterpret_cast<const void *>(&q4_k_gemv_ncol<NC, L, RESIDENT>), kThreads, lds);
    if (oe != hipSuccess) return oe;
    uint32_t per_cu = resident < 1 ? 1u : (uint32_t)resident;
    if (per_cu > 4u) per_cu = 4u;
    uint32_t cap = (uint32_t)ctx->num_cus * per_cu;
    if (blocks > cap) blocks = cap;
    hipLaunchKernelGGL((q4_k_gemv_ncol<NC, L, RESIDENT>), dim3(blocks), dim3(kThreads), lds,
                       ctx->stream, w, x, gain, eps, y, units, rows);
    return hipGetLastError();
}

template <int NC>
hipError_t dispatch_l(lev_ctx *ctx, const uint8_t *w, const float *x, const float *gain, float eps,
                      float *y, uint32_t units, uint32_t rows) {
    if (units > 64) return launch_ncol<NC, 64, false>(ctx, w, x, gain, eps, y, units, rows);
    constexpr bool res = NC <= 2;
    if (units > 32) return launch_ncol<NC, 64, res>(ctx, w, x, gain, eps, y, units, rows);
    if (units > 16) return launch_ncol<NC, 32, res>(ctx, w, x, gain, eps, y, units, rows);
    if (units > 8) return launch_ncol<NC, 16, res>(ctx, w, x, gain, eps, y, units, rows);
    if (units > 4) return launch_ncol<NC, 8, res>(ctx, w, x, gain, eps, y, units, rows);
    return launch_ncol<NC, 4, res>(ctx, w, x, gain, eps, y, units, rows);
}

}  // namespace

// Columns per launch such that the staged activations fit in LDS.
static uint32_t q4k_cols_per_launch(uint32_t in_dim, uint32_t ncol) {
    const uint32_t budget = 144u * 1024u;
    uint32_t per_col = 16u * (in_dim / 64u + 1u) * 16u;
    uint32_t fit = budget / per_col;
    uint32_t nc = ncol < fit ? ncol : fit;
    if (nc >= 8) return 8;
    if (nc >= 4) return 4;
    if (nc == 3) return 3;
    return nc;   // 0 (does not fit), 1 or 2
}

uint32_t lev_q4_k_mfma_cols(const lev_ctx *ctx, uint32_t in_dim);
hipError_t lev_q4_k_mfma_gemv_launch(lev_ctx *ctx, const uint8_t *w, const float *x, const float *gain,
                                     float eps, float *y, uint32_t in_dim, uint32_t rows,
                                     uint32_t ncol);

// Built-in kernel family (1 = integer matrix cores, 0 = vector ALU).  The
// matrix-core kernel forms every dot product without rounding and is the choice
// wherever its activation staging fits; the vector-ALU kernel (f32 FMA chains)
// takes the other shapes and stays a candidate for lev_hip_forge_select.
uint32_t lev_q4_k_mfma_narrow_cols(const lev_ctx *ctx, uint32_t in_dim);

// Whether the matrix-core family takes this shape: its four-columns-per-product kernel up to
// in_dim 8192, its one- and two-column kernel up to in_dim 32768 / ncol.
static bool q4k_mfma_serves(const lev_ctx *ctx, uint32_t in_dim, uint32_t ncol) {
    return lev_q4_k_mfma_cols(ctx, in_dim) != 0u || ncol <= lev_q4_k_mfma_narrow_cols(ctx, in_dim);
}

static uint32_t q4k_builtin_family(const lev_ctx *ctx, uint32_t in_dim, uint32_t rows, uint32_t ncol) {
    (void)rows;
    return q4k_mfma_serves(ctx, in_dim, ncol) ? 1u : 0u;
}

hipError_t lev_q4_k_gemv_launch(lev_ctx *ctx, const uint8_t *w, const float *x, const float *gain,
                                float eps, float *y, uint32_t in_dim, uint32_t rows,
                                uint32_t ncol) {
    const uint32_t units = in_dim / 64u;
    uint32_t done = 0;
    // a schedule installed for this shape (lev_hip_forge_select) overrides the built-in choice
    const lev_schedule *sel = lev_selected(ctx, LEV_OP_Q4_K_GEMV, in_dim, rows, ncol);
    const bool mfma = (sel ? sel->family : q4k_builtin_family(ctx, in_dim, rows, ncol)) == 1u;
    // one column, or two of a row too wide for the four-column kernel: the narrow kernel
    if (mfma && ncol <= lev_q4_k_mfma_narrow_cols(ctx, in_dim) && (ncol == 1u || lev_q4_k_mfma_cols(ctx, in_dim) < ncol))
        return lev_q4_k_mfma_gemv_launch(ctx, w, x, gain, eps, y, in_dim, rows, ncol);
    const uint32_t mfma_cols = mfma ? lev_q4_k_mfma_cols(ctx, in_dim) : 0u;
    while (mfma_cols && done < ncol) {
        uint32_t nc = ncol - done < mfma_cols ? ncol - done : mfma_cols;
        hipError_t e = lev_q4_k_mfma_gemv_launch(ctx, w, x + (uint64_t)done * in_dim, gain, eps,
                                                 y + (uint64_t)done * rows, in_dim, rows, nc);
        if (e != hipSuccess) return e;
        done += nc;
    }
    while (done < ncol) {
        uint32_t nc = q4k_cols_per_launch(in_dim, ncol - done);
        if (nc == 0) return hipErrorInvalidValue;
        const float *xc = x + (uint64_t)done * in_dim;
        float *yc = y + (uint64_t)done * rows;
        hipError_t e;
        switch (nc) {
            case 8: e = dispatch_l<8>(ctx, w, xc, gain, eps, yc, units, rows); break;
            case 4: e = dispatch_l<4>(ctx, w, xc, gain, eps, yc, units, rows); break;
            case 3: e = dispatch_l<3>(ctx, w, xc, gain, eps, yc, units, rows); break;
            case 2: e = dispatch_l<2>(ctx, w, xc, gain, eps, yc, units, rows); break;
            default: e = dispatch_l<1>(ctx, w, xc, gain, eps, yc, units, rows); break;
        }
        if (e != hipSuccess) return e;
        done += nc;
    }
    return hipSuccess;
}

// Candidate schedules of a Q4_K GEMV shape, the built-in choice first
// (schedule::derive, lev-forge/src/schedule.rs:83-105: baseline first, then the
// legal alternatives): the matrix-core kernel where its staging fits, and the
// vector-ALU kernel.
uint32_t lev_q4_k_gemv_candidates(const lev_ctx *ctx, uint32_t in_dim, uint32_t rows, uint32_t ncol,
                                  lev_schedule *out, uint32_t capacity) {
    const uint32_t first = q4k_builtin_family(ctx, in_dim, rows, ncol);
    uint32_t n = 0;
    if (n < capacity) out[n] = lev_schedule{LEV_OP_Q4_K_GEMV, first, 0u, 0u};
    ++n;
    if (q4k_mfma_serves(ctx, in_dim, ncol)) {
        if (n < capacity) out[n] = lev_schedule{LEV_OP_Q4_K_GEMV, 1u - first, 0u, 0u};
        ++n;
    }
    return n;
}

extern "C" int lev_hip_q4_k_gemv_ncol(lev_ctx *ctx, const void *d_w, size_t w_bytes, uint64_t w_off,
                                      const float *d_x, size_t x_count, const float *d_gain,
                                      float eps, float *d_y, size_t y_capacity, uint32_t in_dim,
                                      uint32_t rows, uint32_t ncol) {
    LEV_REQUIRE_CTX(ctx);
    if (ncol == 0 || ncol > LEV_MAX_GEMV_COLUMNS)
        return lev_fail(ctx, LEV_ERR_BAD_DIMENSIONS, "q4_k_gemv_ncol: %u columns (1..%d)", ncol,
                        LEV_MAX_GEMV_COLUMNS);
    if (d_gain && !(eps >= 0.f))
        return lev_fail(ctx, LEV_ERR_BAD_DIMENSIONS, "q4_k_gemv_ncol: eps %g", (double)eps);
    lev_geom g;
    int st = lev_check_matvec(ctx, "q4_k_gemv_ncol", 256, 144, d_w, w_bytes, w_off, d_x, x_count,
                              (uint64_t)in_dim * ncol, d_y, y_capacity, (uint64_t)rows * ncol,
                              in_dim, rows, &g);
    if (st != LEV_OK) return st;
    const uint8_t *w = static_cast<const uint8_t *>(d_w) + w_off;
    if ((reinterpret_cast<uintptr_t>(w) & 15u) || (reinterpret_cast<uintptr_t>(d_x) & 15u) ||
        (d_gain && (reinterpret_cast<uintptr_t>(d_gain) & 15u)))
        return lev_fail(ctx, LEV_ERR_BAD_DIMENSIONS,
                        "q4_k_gemv_ncol: weights, x and gain must be 16-byte aligned");
    if (q4k_cols_per_launch(in_dim, 1) == 0)
        return lev_fail(ctx, LEV_ERR_EXCEEDS_MODEL_WORKLOAD,
                        "q4_k_gemv_ncol: inDim %u does not fit the activation staging", in_dim);
    return lev_hip_check(ctx, lev_q4_k_gemv_launch(ctx, w, d_x, d_gain, eps, d_y, in_dim, rows, ncol),
                         "q4_k_gemv_ncol launch");
}

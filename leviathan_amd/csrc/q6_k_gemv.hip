// Q6_K decode GEMV (+ greedy-token epilogue) for gfx950.
//
// Stands in for g4_q6_matvec / _tiled / _coop (Gemma4.swift:4065, 4109;
// Q6Cooperative.swift:54-98), the GLSL q6k.matvec (lev-forge/src/q6k.rs:61-187)
// and the argmax step (lev-forge/src/ops.rs:479-516).
//
// Layout in HBM is the GGUF one: 210-byte superblocks of 256 weights
// (ql[128] low nibbles, qh[64] 2-bit tops, 16 int8 sub-scales, fp16 d;
// Q6.swift:4-62), 2-byte aligned.
//
// Work unit: 32 weights = 16 ql bytes + the 16 qh bytes they pair with.
// Unit g of a row (g = 8*superblock + 4*half + v, v = 0..3) owns
//   ql[64*half + 16*v .. +16)      low nibbles -> elements  E..E+15
//                                  high nibbles -> elements E+64..E+79
//   qh[32*half + 16*(v&1) .. +16)  bit pairs (v>>1)*2 and (v>>1)*2+4
// with E = 128*half + 16*v inside the superblock, so both of its 16-element
// groups have ONE sub-scale each (scales[8*half + (v&1) + 2*(v>>1)] and +4).
// A lane keeps the 32 activations of its unit(s) in registers for every row
// it visits; the -32 offset is folded out:  sc*(sum q*x - 32*sum x).
// The 6-bit codes are assembled four per dword with byte-wise logic, turned
// into fp16 subnormals (q * 2^-24) by masking and fed to v_fma_mix_f32.
#include "lev_common.hpp"

namespace {

constexpr int kThreads = 512;
constexpr int kWaves = kThreads / LEV_WAVE;

struct __attribute__((packed, aligned(2))) u32x4_a2 { uint32_t v[4]; };
struct __attribute__((packed, aligned(2))) u32x2_a2 { uint32_t v[2]; };

struct q6_unit_x {
    lev_f32x4 lo[4];   // elements E..E+15
    lev_f32x4 hi[4];   // elements E+64..E+79
    float sum_lo, sum_hi;
};

struct q6_unit_w {
    uint32_t ql[4];
    uint32_t qh[4];
    uint32_t sc[2];    // the 8 sub-scale bytes of the unit's half
    uint32_t d;        // fp16 bits
};

__device__ __forceinline__ void q6_load_unit(const uint8_t *row, uint32_t g, q6_unit_w &u) {
    const uint32_t sb = g >> 3, half = (g >> 2) & 1u, v = g & 3u;
    const uint8_t *blk = row + (uint64_t)sb * 210u;
    u32x4_a2 a = *reinterpret_cast<const u32x4_a2 *>(blk + 64u * half + 16u * v);
    u32x4_a2 b = *reinterpret_cast<const u32x4_a2 *>(blk + 128u + 32u * half + 16u * (v & 1u));
    u32x2_a2 c = *reinterpret_cast<const u32x2_a2 *>(blk + 192u + 8u * half);
    u.d = *reinterpret_cast<const uint16_t *>(blk + 208u);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        u.ql[i] = a.v[i];
        u.qh[i] = b.v[i];
    }
    u.sc[0] = c.v[0];
    u.sc[1] = c.v[1];
}

// sum_i code_i * x_i over four code bytes packed in `c`, scaled by 2^-24.
__device__ __forceinline__ float q6_dot4(uint32_t c, lev_f32x4 x, float acc) {
    lev_f16x2 e02 = __builtin_bit_cast(lev_f16x2, c & 0x00FF00FFu);
    lev_f16x2 e13 = __builtin_bit_cast(lev_f16x2, (c >> 8) & 0x00FF00FFu);
    acc = fmaf((float)e02.x, x.x, acc);
    acc = fmaf((float)e13.x, x.y, acc);
    acc = fmaf((float)e02.y, x.z, acc);
    acc = fmaf((float)e13.y, x.w, acc);
    return acc;
}

// Contribution of one unit to its row's dot product.  `v` = g & 3.
__device__ __forceinline__ float q6_unit_dot(const q6_unit_w &u, const q6_unit_x &x, uint32_t v) {
    const uint32_t pair = v >> 1;              // 0: qh bit pairs 0 and 4, 1: pairs 2 and 6
    const uint32_t shl = 4u - 2u * pair;       // (qh << shl) & 0x30 -> top bits of the low set
    const uint32_t shr = 2u * pair;            // (qh >> shr) & 0x30 -> top bits of the high set
    float lo = 0.f, hi = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        uint32_t q = u.ql[i], h = u.qh[i];
        uint32_t cl = (q & 0x0F0F0F0Fu) | ((h << shl) & 0x30303030u);
        uint32_t ch = ((q >> 4) & 0x0F0F0F0Fu) | ((h >> shr) & 0x30303030u);
        lo = q6_dot4(cl, x.lo[i], lo);
        hi = q6_dot4(ch, x.hi[i], hi);
    }
    // sub-scales: byte (v&1) + 2*pair for the low set, +4 for the high set
    const uint32_t bi = (v & 1u) + 2u * pair;
    float s_lo = (float)(int)__builtin_amdgcn_sbfe((int)u.sc[0], 8u * bi, 8u);
    float s_hi = (float)(int)__builtin_amdgcn_sbfe((int)u.sc[1], 8u * bi, 8u);
    float d = lev_f16_bits_to_f32(u.d);
    float t = fmaf(s_lo, fmaf(lo, 16777216.0f, -32.0f * x.sum_lo),
                   s_hi * fmaf(hi, 16777216.0f, -32.0f * x.sum_hi));
    return d * t;
}

// LDS layout of the activations: float4 slot q*(U+1)+g, q = 0..3 low set,
// 4..7 high set of unit g; U = units per row.
__device__ __forceinline__ void q6_stage_x(const float *__restrict__ x, lev_f32x4 *xs,
                                           uint32_t units, uint32_t tid) {
    const lev_f32x4 *x4 = reinterpret_cast<const lev_f32x4 *>(x);
    const uint32_t n4 = units * 8u;
    for (uint32_t i = tid; i < n4; i += kThreads) {
        uint32_t e = i * 4u;
        uint32_t c = e >> 7, r = e & 127u;
        uint32_t g = 4u * c + ((r & 63u) >> 4);
        uint32_t q = 4u * (r >> 6) + ((r & 15u) >> 2);
        xs[q * (units + 1u) + g] = x4[i];
    }
}

__device__ __forceinline__ void q6_fetch_x(const lev_f32x4 *xs, uint32_t units, uint32_t g,
                                           q6_unit_x &x) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        x.lo[q] = xs[q * (units + 1u) + g];
        x.hi[q] = xs[(4 + q) * (units + 1u) + g];
    }
    float a = 0.f, b = 0.f;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        a += (x.lo[q].x + x.lo[q].y) + (x.lo[q].z + x.lo[q].w);
        b += (x.hi[q].x + x.hi[q].y) + (x.hi[q].z + x.hi[q].w);
    }
    x.sum_lo = a;
    x.sum_hi = b;
}

// ---- argmax + margin (lev-forge/src/ops.rs:479-516) ------------------------

struct top2 {
    float best, second;
    uint32_t idx;
};

__device__ __forceinline__ top2 top2_merge(top2 a, top2 b) {
    // take b when strictly larger, or equal with the lower index (ops.rs:508)
    bool take = b.best > a.best || (b.best == a.best && b.idx < a.idx);
    top2 r;
    r.best = take ? b.best : a.best;
    r.idx = take ? b.idx : a.idx;
    float other = take ? fmaxf(a.best, b.second) : fmaxf(b.best, a.second);
    r.second = fmaxf(other, take ? a.second : b.second);
    return r;
}


__device__ __forceinline__ top2 top2_wave(top2 m) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        top2 o;
        o.best = __shfl_xor(m.best, off);
        o.second = __shfl_xor(m.second, off);
        o.idx = __shfl_xor(m.idx, off);
        m = top2_merge(m, o);
    }
    return m;
}

constexpr float kTop2Floor = -INFINITY;

template <int L, int P>
__device__ __forceinline__ void q6_load_row(const uint8_t *__restrict__ w, uint64_t row_bytes,
                                            uint32_t row, uint32_t rows, uint32_t lu,
                                            uint32_t units, q6_unit_w (&W)[P]) {
    // Lanes past the end of the matrix read a valid unit (clamped) and have
    // their block scale forced to zero: no divergent control flow around loads.
    const uint32_t row_c = row < rows ? row : rows - 1u;
#pragma unroll
    for (int p = 0; p < P; ++p) {
        uint32_t g = lu + p * L;
        const bool ok = row < rows && g < units;
        q6_load_unit(w + row_c * row_bytes, g < units ? g : units - 1u, W[p]);
        W[p].d = ok ? W[p].d : 0u;
    }
}

template <int L, int P>
__device__ __forceinline__ void q6_finish_row(float *__restrict__ y, uint32_t row, uint32_t rows,
                                              uint32_t lu, const q6_unit_w (&W)[P],
                                              const q6_unit_x (&X)[P], top2 &m) {
    float acc = 0.f;
#pragma unroll
    for (int p = 0; p < P; ++p) acc += q6_unit_dot(W[p], X[p], (lu + p * L) & 3u);
    acc = lev_group_sum<L>(acc);
    if (lu % L == L - 1 && row < rows) {
        y[row] = acc;
        // running top two of the rows this lane finishes (rows ascend, so a
        // tie keeps the earlier, lower index)
        if (acc > m.best) {
            m.second = m.best;
            m.best = acc;
            m.idx = row;
        } else if (acc > m.second) {
            m.second = acc;
        }
    }
}

// L lanes per row-part, P passes of L units, S waves share a row (units <=
// S*L*P; S > 1 only with L = 64): with S = 2 a 4096-wide row costs each lane
// one unit instead of two, which brings the kernel under 128 VGPRs and five
// waves per SIMD instead of three.  Persistent workgroups, weights
// double-buffered.
// partials (optional): the workgroup's top two logits and the index of the
// best, one float4 {best, second, idx bits, 0} per workgroup, for the greedy
// token epilogue.
template <int L, int P, int S>
__global__ void __launch_bounds__(kThreads)
q6_k_gemv_units(const uint8_t *__restrict__ w, const float *__restrict__ x, float *__restrict__ y,
                uint32_t units, uint32_t rows, lev_f32x4 *__restrict__ partials) {
    extern __shared__ lev_f32x4 xs[];
    constexpr int G = LEV_WAVE / L;
    constexpr uint32_t kRowsPerTile = kWaves * G / S;
    static_assert(S == 1 || L == LEV_WAVE, "rows are shared by whole waves only");
    __shared__ float part[2][S > 1 ? kWaves : 1];
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & (LEV_WAVE - 1);
    const uint32_t wave = tid / LEV_WAVE;
    const uint32_t grp = lane / L;
    const uint32_t lu = (wave % S) * (L * P) + lane % L;   // first unit of this lane
    const uint64_t row_bytes = (uint64_t)(units >> 3) * 210u;
    const uint32_t in_tile = (wave / S) * G + grp;
    const uint32_t step = gridDim.x * kRowsPerTile;

    uint32_t base = blockIdx.x * kRowsPerTile;
    if (base >= rows) return;   // never: the grid has at most one workgroup per tile

    top2 m{kTop2Floor, kTop2Floor, 0xFFFFFFFFu};
    q6_unit_w Wa[P], Wb[P];
    q6_load_row<L, P>(w, row_bytes, base + in_tile, rows, lu, units, Wa);
    q6_stage_x(x, xs, units, tid);
    __syncthreads();

    q6_unit_x X[P];
#pragma unroll
    for (int p = 0; p < P; ++p) {
        uint32_t g = lu + p * L;
        if (g < units) {
            q6_fetch_x(xs, units, g, X[p]);
        } else {
#pragma unroll
            for (int q = 0; q < 4; ++q) X[p].lo[q] = X[p].hi[q] = lev_f32x4{0.f, 0.f, 0.f, 0.f};
            X[p].sum_lo = X[p].sum_hi = 0.f;
        }
    }

    // The prefetch is unconditional (clamped past the end): a branch around the
    // loads would make the compiler wait for them before the current row is used.
    uint32_t buf = 0;
    auto finish = [&](uint32_t row0, const q6_unit_w (&W)[P]) {
        if constexpr (S == 1) {
            q6_finish_row<L, P>(y, row0 + in_tile, rows, lu, W, X, m);
        } else {
            // the S waves of a row leave their parts in LDS; one thread per row
            // adds them in wave order.  Two part buffers: one barrier per tile.
            float acc = 0.f;
#pragma unroll
            for (int p = 0; p < P; ++p) acc += q6_unit_dot(W[p], X[p], (lu + p * L) & 3u);
            acc = lev_group_sum<L>(acc);
            if (lane == LEV_WAVE - 1) part[buf][wave] = acc;
            __syncthreads();
            if (tid < kRowsPerTile && row0 + tid < rows) {
                float sum = part[buf][tid * S];
#pragma unroll
                for (int k = 1; k < S; ++k) sum += part[buf][tid * S + k];
                y[row0 + tid] = sum;
                if (sum > m.best) {
                    m.second = m.best;
                    m.best = sum;
                    m.idx = row0 + tid;
                } else if (sum > m.second) {
                    m.second = sum;
                }
            }
            buf ^= 1u;
        }
    };
    while (true) {
        uint32_t next = base + step;
        q6_load_row<L, P>(w, row_bytes, next + in_tile, rows, lu, units, Wb);
        finish(base, Wa);
        if (next >= rows) break;
        base = next;
        next = base + step;
        q6_load_row<L, P>(w, row_bytes, next + in_tile, rows, lu, units, Wa);
        finish(base, Wb);
        if (next >= rows) break;
        base = next;
    }
    if (partials) {
        __shared__ float s_best[kWaves], s_second[kWaves];
        __shared__ uint32_t s_idx[kWaves];
        m = top2_wave(m);
        if (lane == 0) {
            s_best[wave] = m.best;
            s_second[wave] = m.second;
            s_idx[wave] = m.idx;
        }
        __syncthreads();
        if (tid == 0) {
            top2 r{s_best[0], s_second[0], s_idx[0]};
            for (int k = 1; k < kWaves; ++k) r = top2_merge(r, top2{s_best[k], s_second[k], s_idx[k]});
            partials[blockIdx.x] = lev_f32x4{r.best, r.second, __builtin_bit_cast(float, r.idx), 0.f};
        }
    }
}

// One workgroup: merges the per-workgroup partials of the GEMV.
__global__ void __launch_bounds__(256)
argmax_partials_kernel(const lev_f32x4 *__restrict__ partials, uint32_t n,
                       uint32_t *__restrict__ out_idx, float *__restrict__ out_margin) {
    __shared__ float s_best[4], s_second[4];
    __shared__ uint32_t s_idx[4];
    const uint32_t t = threadIdx.x;
    top2 m{kTop2Floor, kTop2Floor, 0xFFFFFFFFu};
    for (uint32_t i = t; i < n; i += 256u) {
        lev_f32x4 p = partials[i];
        const float idx_bits = p.z;   // a copy: bit_cast straight from a vector element reads element 0
        m = top2_merge(m, top2{p.x, p.y, __float_as_uint(idx_bits)});
    }
    m = top2_wave(m);
    if ((t & 63u) == 0) {
        s_best[t >> 6] = m.best;
        s_second[t >> 6] = m.second;
        s_idx[t >> 6] = m.idx;
    }
    __syncthreads();
    if (t == 0) {
        top2 r{s_best[0], s_second[0], s_idx[0]};
        for (int k = 1; k < 4; ++k) r = top2_merge(r, top2{s_best[k], s_second[k], s_idx[k]});
        if (out_idx) out_idx[0] = r.idx == 0xFFFFFFFFu ? 0u : r.idx;   // nothing above -inf: first
        if (out_margin) out_margin[0] = r.best - r.second;
    }
}

// Any in_dim: one wave per row, activations read through the cache.
__global__ void __launch_bounds__(kThreads)
q6_k_gemv_generic(const uint8_t *__restrict__ w, const float *__restrict__ x,
                  float *__restrict__ y, uint32_t units, uint32_t rows) {
    const uint32_t lane = threadIdx.x & (LEV_WAVE - 1);
    const uint32_t row = blockIdx.x * kWaves + threadIdx.x / LEV_WAVE;
    if (row >= rows) return;
    const uint8_t *rp = w + (uint64_t)row * (units >> 3) * 210u;
    float acc = 0.f;
    for (uint32_t g = lane; g < units; g += LEV_WAVE) {
        q6_unit_w u;
        q6_load_unit(rp, g, u);
        q6_unit_x ux;
        const float *xb = x + (uint64_t)(g >> 2) * 128u + 16u * (g & 3u);
        float a = 0.f, b = 0.f;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            ux.lo[q] = lev_f32x4{xb[4 * q], xb[4 * q + 1], xb[4 * q + 2], xb[4 * q + 3]};
            ux.hi[q] = lev_f32x4{xb[64 + 4 * q], xb[65 + 4 * q], xb[66 + 4 * q], xb[67 + 4 * q]};
            a += (ux.lo[q].x + ux.lo[q].y) + (ux.lo[q].z + ux.lo[q].w);
            b += (ux.hi[q].x + ux.hi[q].y) + (ux.hi[q].z + ux.hi[q].w);
        }
        ux.sum_lo = a;
        ux.sum_hi = b;
        acc += q6_unit_dot(u, ux, g & 3u);
    }
    acc = lev_group_sum<64>(acc);
    if (lane == LEV_WAVE - 1) y[row] = acc;
}

__global__ void __launch_bounds__(1024)
argmax_kernel(const float *__restrict__ logits, uint32_t vocab, uint32_t *__restrict__ out_idx,
              float *__restrict__ out_margin) {
    __shared__ float s_best[16], s_second[16];
    __shared__ uint32_t s_idx[16];
    const float *l = logits + (uint64_t)blockIdx.x * vocab;
    const uint32_t t = threadIdx.x;
    top2 m{kTop2Floor, kTop2Floor, 0xFFFFFFFFu};
    for (uint32_t i = t; i < vocab; i += 1024) {
        float v = l[i];
        if (v > m.best) {
            m.second = m.best;
            m.best = v;
            m.idx = i;
        } else if (v > m.second) {
            m.second = v;
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        top2 o;
        o.best = __shfl_xor(m.best, off);
        o.second = __shfl_xor(m.second, off);
        o.idx = __shfl_xor(m.idx, off);
        m = top2_merge(m, o);
    }
    if ((t & 63u) == 0) {
        s_best[t >> 6] = m.best;
        s_second[t >> 6] = m.second;
        s_idx[t >> 6] = m.idx;
    }
    __syncthreads();
    if (t == 0) {
        top2 r{s_best[0], s_second[0], s_idx[0]};
        for (int k = 1; k < 16; ++k) r = top2_merge(r, top2{s_best[k], s_second[k], s_idx[k]});
        if (out_idx) out_idx[blockIdx.x] = r.idx == 0xFFFFFFFFu ? 0u : r.idx;
        if (out_margin) out_margin[blockIdx.x] = r.best - r.second;
    }
}

template <int L, int P, int S = 1>
hipError_t launch_units(lev_ctx *ctx, const uint8_t *w, const float *x, float *y, uint32_t units,
                        uint32_t rows, uint32_t *d_argmax, float *d_margin) {
    constexpr uint32_t rows_per_tile = kWaves * (LEV_WAVE / L) / S;
    uint32_t blocks = (rows + rows_per_tile - 1) / rows_per_tile;
    size_t lds = (size_t)8 * (units + 1) * sizeof(lev_f32x4);
    // persistent grid: exactly the workgroups that are resident at once, so
    // that no workgroup waits for a slot behind another one's whole loop
    int per_cu = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, q6_k_gemv_units<L, P, S>, kThreads, lds) !=
            hipSuccess || per_cu < 1)
        per_cu = 2;
    uint32_t cap = (uint32_t)ctx->num_cus * (uint32_t)per_cu;
    if (blocks > cap) blocks = cap;
    lev_f32x4 *partials = nullptr;
    if (d_argmax || d_margin) {
        // one partial per workgroup, in the context's fixed buffer
        if (blocks > lev_ctx::kArgmaxPartials) blocks = lev_ctx::kArgmaxPartials;
        partials = static_cast<lev_f32x4 *>(ctx->argmax_partials);
    }
    hipLaunchKernelGGL((q6_k_gemv_units<L, P, S>), dim3(blocks), dim3(kThreads), lds, ctx->stream, w, x,
                       y, units, rows, partials);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess || !partials) return e;
    hipLaunchKernelGGL(argmax_partials_kernel, dim3(1), dim3(256), 0, ctx->stream, partials, blocks,
                       d_argmax, d_margin);
    return hipGetLastError();
}

}  // namespace

// GEMV with the greedy-token epilogue: d_argmax / d_margin may be NULL.
hipError_t lev_q6_k_gemv_argmax_launch(lev_ctx *ctx, const uint8_t *w, const float *x, float *y,
                                       uint32_t in_dim, uint32_t rows, uint32_t *d_argmax,
                                       float *d_margin) {
    const uint32_t units = in_dim / 32u;   // 8 per superblock
    const bool fast = ((reinterpret_cast<uintptr_t>(w) & 1u) == 0u) &&
                      ((reinterpret_cast<uintptr_t>(x) & 15u) == 0u) && units <= 256u;
    if (!fast) {
        uint32_t blocks = (rows + kWaves - 1) / kWaves;
        hipLaunchKernelGGL(q6_k_gemv_generic, dim3(blocks), dim3(kThreads), 0, ctx->stream, w, x, y,
                           units, rows);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess || (!d_argmax && !d_margin)) return e;
        hipLaunchKernelGGL(argmax_kernel, dim3(1), dim3(1024), 0, ctx->stream, y, rows, d_argmax,
                           d_margin);
        return hipGetLastError();
    }
    if (units > 192) return launch_units<64, 4>(ctx, w, x, y, units, rows, d_argmax, d_margin);
    if (units > 128) return launch_units<64, 3>(ctx, w, x, y, units, rows, d_argmax, d_margin);
    if (units > 64) return launch_units<64, 1, 2>(ctx, w, x, y, units, rows, d_argmax, d_margin);
    if (units > 32) return launch_units<64, 1>(ctx, w, x, y, units, rows, d_argmax, d_margin);
    if (units > 16) return launch_units<32, 1>(ctx, w, x, y, units, rows, d_argmax, d_margin);
    if (units > 8) return launch_units<16, 1>(ctx, w, x, y, units, rows, d_argmax, d_margin);
    return launch_units<8, 1>(ctx, w, x, y, units, rows, d_argmax, d_margin);
}

hipError_t lev_q6_k_gemv_launch(lev_ctx *ctx, const uint8_t *w, const float *x, float *y,
                                uint32_t in_dim, uint32_t rows) {
    return lev_q6_k_gemv_argmax_launch(ctx, w, x, y, in_dim, rows, nullptr, nullptr);
}

hipError_t lev_argmax_launch(lev_ctx *ctx, const float *logits, uint32_t vocab, uint32_t ncol,
                             uint32_t *idx, float *margin) {
    hipLaunchKernelGGL(argmax_kernel, dim3(ncol), dim3(1024), 0, ctx->stream, logits, vocab, idx,
                       margin);
    return hipGetLastError();
}

extern "C" int lev_hip_q6_k_gemv(lev_ctx *ctx, const void *d_w, size_t w_bytes, uint64_t w_off,
                                 const float *d_x, size_t x_count, float *d_y, size_t y_capacity,
                                 uint32_t in_dim, uint32_t out_rows, uint32_t *d_argmax,
                                 float *d_margin) {
    LEV_REQUIRE_CTX(ctx);
    lev_geom g;
    int st = lev_check_matvec(ctx, "q6_k_gemv", 256, 210, d_w, w_bytes, w_off, d_x, x_count, in_dim,
                              d_y, y_capacity, out_rows, in_dim, out_rows, &g);
    if (st != LEV_OK) return st;
    const uint8_t *w = static_cast<const uint8_t *>(d_w) + w_off;
    return lev_hip_check(ctx,
                         lev_q6_k_gemv_argmax_launch(ctx, w, d_x, d_y, in_dim, out_rows, d_argmax,
                                                     d_margin),
                         "q6_k_gemv launch");
}

extern "C" int lev_hip_argmax(lev_ctx *ctx, const float *d_logits, uint32_t vocab, uint32_t ncol,
                              uint32_t *d_index, float *d_margin) {
    LEV_REQUIRE_CTX(ctx);
    if (!d_logits || (!d_index && !d_margin))
        return lev_fail(ctx, LEV_ERR_INVALID_ARGUMENT, "argmax: null pointer");
    if (vocab == 0 || ncol == 0 || ncol > 65535u)
        return lev_fail(ctx, LEV_ERR_BAD_DIMENSIONS, "argmax: vocab %u, columns %u", vocab, ncol);
    return lev_hip_check(ctx, lev_argmax_launch(ctx, d_logits, vocab, ncol, d_index, d_margin),
                         "argmax launch");
}

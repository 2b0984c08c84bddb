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
// groups have ONE sub-scale each (scales[8*half + v] and [8*half + 4 + v]).
//
// Arithmetic.  Logits are sums of 4096 terms that cancel from magnitudes of
// several thousand down to O(1), and the gate is 1e-4 of max(1, |logit|): f32
// accumulation sits at that bound whatever the order.  So the products are
// formed EXACTLY, on integers: while staging, every 16-element group of x is
// written as 27-bit integers X_i = rint(x_i * 2^(26-e)), 2^e > max|x| of the
// group (exact for every element within 2^-3 of the group's maximum, 2^-27 of the
// maximum otherwise), split into four balanced 7-bit digits held as int8
//   X = l0*2^21 + l1*2^14 + l2*2^7 + l3,
// and the 6-bit codes, assembled four per dword with byte-wise logic, go
// straight into v_dot4_i32_i8 against each digit plane: four exact int32 dot
// products per group, recombined in f64.  The -32 offset comes out through the
// group's exact integer sum.  Scales, the sum over a row and the reduction
// across lanes are f64; the result is rounded to f32 once.  A lane keeps the
// digit planes of its unit(s) in registers for every row it visits.
#include "lev_common.hpp"
#include "top2.hpp"

#include <cstdlib>

namespace {

constexpr int kThreads = 512;
constexpr int kWaves = kThreads / LEV_WAVE;
#ifndef LEV_Q6_DEPTH
#define LEV_Q6_DEPTH 3   // tiles in flight per wave of the one-unit-per-lane kernels
#endif

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

// ---- f32 path of the generic kernel (any geometry, activations from global memory) ----

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

// Contribution of one unit to its row's dot product.  `v` = g & 3.  The two
// 16-element sums are f32 (two chains each), everything behind them f64.
__device__ __forceinline__ double q6_unit_dot(const q6_unit_w &u, const q6_unit_x &x, uint32_t v) {
    const uint32_t pair = v >> 1;              // 0: qh bit pairs 0 and 4, 1: pairs 2 and 6
    const uint32_t shl = 4u - 2u * pair;       // (qh << shl) & 0x30 -> top bits of the low set
    const uint32_t shr = 2u * pair;            // (qh >> shr) & 0x30 -> top bits of the high set
    float lo0 = 0.f, lo1 = 0.f, hi0 = 0.f, hi1 = 0.f;
#pragma unroll
    for (int i = 0; i < 4; i += 2) {
        uint32_t q = u.ql[i], h = u.qh[i];
        lo0 = q6_dot4((q & 0x0F0F0F0Fu) | ((h << shl) & 0x30303030u), x.lo[i], lo0);
        hi0 = q6_dot4(((q >> 4) & 0x0F0F0F0Fu) | ((h >> shr) & 0x30303030u), x.hi[i], hi0);
        q = u.ql[i + 1], h = u.qh[i + 1];
        lo1 = q6_dot4((q & 0x0F0F0F0Fu) | ((h << shl) & 0x30303030u), x.lo[i + 1], lo1);
        hi1 = q6_dot4(((q >> 4) & 0x0F0F0F0Fu) | ((h >> shr) & 0x30303030u), x.hi[i + 1], hi1);
    }
    // sub-scales: byte v of the half's low four for the low set, of its high four for the high set
    const double s_lo = (double)(int)__builtin_amdgcn_sbfe((int)u.sc[0], 8u * v, 8u);
    const double s_hi = (double)(int)__builtin_amdgcn_sbfe((int)u.sc[1], 8u * v, 8u);
    const double t_lo = fma(((double)lo0 + (double)lo1), 16777216.0, -32.0 * (double)x.sum_lo);
    const double t_hi = fma(((double)hi0 + (double)hi1), 16777216.0, -32.0 * (double)x.sum_hi);
    return (double)lev_f16_bits_to_f32(u.d) * fma(s_lo, t_lo, s_hi * t_hi);
}

// ---- exact path ------------------------------------------------------------

// Digit planes of one unit: lo[i] / hi[i] hold, for elements 4i..4i+3 of the
// low / high set, the four dwords {l0, l1, l2, l3} of packed int8 digits.
struct q6_unit_xi {
    lev_u32x4 lo[4];
    lev_u32x4 hi[4];
};

// Per 16-element group of x: p = 2^(e-26) and sx = sum of the group's integers X_i.
struct q6_group_meta {
    double p, sx;
};

// LDS: uint4 slot q*(U+1)+g holds the digit dwords of quad q (0..3 low set,
// 4..7 high set) of unit g; then 2*U group records, group j = element / 16.
__host__ __device__ constexpr size_t q6_lds_bytes(uint32_t units) {
    return (size_t)8 * (units + 1u) * sizeof(lev_u32x4) + (size_t)2 * units * sizeof(q6_group_meta);
}

// Returns false (workgroup-uniform) when x holds a NaN or an infinity.
__device__ __forceinline__ bool q6_stage_digits(const float *__restrict__ x, lev_u32x4 *xs,
                                                q6_group_meta *meta, uint32_t units, uint32_t tid) {
    const lev_f32x4 *x4 = reinterpret_cast<const lev_f32x4 *>(x);
    const uint32_t n4 = units * 8u;
    bool finite = true;
    // whole passes: the four lanes of a group exchange their maxima and sums by DPP
    for (uint32_t base = 0; base < n4; base += kThreads) {
        const uint32_t i = base + tid;
        const bool live = i < n4;
        const lev_f32x4 v = x4[live ? i : n4 - 1u];
        float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
#define LEV_Q6_MAXSTEP(CTRL)                                                                     \
        amax = fmaxf(amax, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(                 \
                               __builtin_bit_cast(int, amax), __builtin_bit_cast(int, amax), CTRL, 0xF, 0xF, false)))
        LEV_Q6_MAXSTEP(0xB1);   // quad_perm [1,0,3,2]
        LEV_Q6_MAXSTEP(0x4E);   // quad_perm [2,3,0,1]
#undef LEV_Q6_MAXSTEP
        uint32_t ex = __float_as_uint(amax) >> 23;          // biased exponent: amax < 2^(ex-126)
        finite = finite && ex != 255u && !(v.x != v.x || v.y != v.y || v.z != v.z || v.w != v.w);
        ex = ex < 25u ? 25u : (ex > 254u ? 254u : ex);      // keeps the scale 2^(152-ex) a normal number
        const float scale = __uint_as_float((279u - ex) << 23);
        int X[4] = {(int)rintf(v.x * scale), (int)rintf(v.y * scale), (int)rintf(v.z * scale),
                    (int)rintf(v.w * scale)};
        int sum = (X[0] + X[1]) + (X[2] + X[3]);            // |X| <= 2^26: sixteen of them fit
        sum += __builtin_amdgcn_update_dpp(0, sum, 0xB1, 0xF, 0xF, false);
        sum += __builtin_amdgcn_update_dpp(0, sum, 0x4E, 0xF, 0xF, false);
        uint32_t dw[4] = {0u, 0u, 0u, 0u};                  // dw[3] = lowest digit l3 ... dw[0] = l0
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            int r = X[k];
#pragma unroll
            for (int dgt = 3; dgt >= 1; --dgt) {
                const int l = __builtin_amdgcn_sbfe(r, 0u, 7u);   // signed low 7 bits: r - l is a multiple of 128
                r = (r - l) >> 7;
                dw[dgt] |= ((uint32_t)l & 0xFFu) << (8 * k);
            }
            dw[0] |= ((uint32_t)r & 0xFFu) << (8 * k);            // |r| <= 33
        }
        if (live) {
            const uint32_t e = i * 4u;
            const uint32_t c = e >> 7, rr = e & 127u;
            const uint32_t g = 4u * c + ((rr & 63u) >> 4);
            const uint32_t q = 4u * (rr >> 6) + ((rr & 15u) >> 2);
            xs[q * (units + 1u) + g] = lev_u32x4{dw[0], dw[1], dw[2], dw[3]};
            if ((i & 3u) == 3u) {
                q6_group_meta m;
                m.p = __hiloint2double((int)((ex + 871u) << 20), 0);   // 2^(ex-152)
                m.sx = (double)sum;
                meta[i >> 2] = m;
            }
        }
    }
    // every wave leaves its verdict in LDS; the barrier waits for LDS traffic only, so the
    // first tile's weight loads (already requested) stay in flight across it
    __shared__ uint32_t s_finite[kWaves];
    const bool wave_ok = __ballot(!finite) == 0ull;
    if ((tid & (LEV_WAVE - 1)) == 0) s_finite[tid / LEV_WAVE] = wave_ok ? 1u : 0u;
    lev_barrier_lds();
    bool all_ok = true;
#pragma unroll
    for (int k = 0; k < kWaves; ++k) all_ok = all_ok && s_finite[k] != 0u;
    return all_ok;
}

__device__ __forceinline__ void q6_fetch_digits(const lev_u32x4 *xs, const q6_group_meta *meta,
                                                uint32_t units, uint32_t g, q6_unit_xi &x,
                                                q6_group_meta &mlo, q6_group_meta &mhi) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        x.lo[q] = xs[q * (units + 1u) + g];
        x.hi[q] = xs[(4 + q) * (units + 1u) + g];
    }
    const uint32_t j = 8u * (g >> 2) + (g & 3u);
    mlo = meta[j];
    mhi = meta[j + 4u];
}

// sum over a 16-element group of code * X, exact.
__device__ __forceinline__ double q6_group_dot(const uint32_t c[4], const lev_u32x4 x[4]) {
    int d0 = 0, d1 = 0, d2 = 0, d3 = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        d0 = __builtin_amdgcn_sdot4((int)c[i], (int)x[i].x, d0, false);
        d1 = __builtin_amdgcn_sdot4((int)c[i], (int)x[i].y, d1, false);
        d2 = __builtin_amdgcn_sdot4((int)c[i], (int)x[i].z, d2, false);
        d3 = __builtin_amdgcn_sdot4((int)c[i], (int)x[i].w, d3, false);
    }
    // |d_k| <= 16*63*64: the pairs fit 32 bits, the whole sum fits f64
    return fma((double)((d0 << 7) + d1), 16384.0, (double)((d2 << 7) + d3));
}

__device__ __forceinline__ double q6_unit_dot_exact(const q6_unit_w &u, const q6_unit_xi &x,
                                                    const q6_group_meta &mlo, const q6_group_meta &mhi,
                                                    uint32_t v) {
    const uint32_t pair = v >> 1;
    const uint32_t shl = 4u - 2u * pair, shr = 2u * pair;
    uint32_t cl[4], ch[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t q = u.ql[i], h = u.qh[i];
        cl[i] = (q & 0x0F0F0F0Fu) | ((h << shl) & 0x30303030u);
        ch[i] = ((q >> 4) & 0x0F0F0F0Fu) | ((h >> shr) & 0x30303030u);
    }
    const double t_lo = fma(-32.0, mlo.sx, q6_group_dot(cl, x.lo));   // sum (code - 32) * X
    const double t_hi = fma(-32.0, mhi.sx, q6_group_dot(ch, x.hi));
    const double s_lo = (double)(int)__builtin_amdgcn_sbfe((int)u.sc[0], 8u * v, 8u) * mlo.p;
    const double s_hi = (double)(int)__builtin_amdgcn_sbfe((int)u.sc[1], 8u * v, 8u) * mhi.p;
    return (double)lev_f16_bits_to_f32(u.d) * fma(s_lo, t_lo, s_hi * t_hi);
}

// ---- argmax + margin (lev-forge/src/ops.rs:479-516) ------------------------


template <int L, int P>
__device__ __forceinline__ void q6_load_row(const uint8_t *__restrict__ w, uint64_t row_bytes,
                                            uint32_t row, uint32_t rows, uint32_t lu,
                                            uint32_t units, q6_unit_w (&W)[P]) {
    // Lanes past the end of the matrix read a valid unit (clamped) and have
    // their block scale forced to zero: no divergent control flow around loads.
    uint32_t row_c = row < rows ? row : rows - 1u;
    // a whole wave per row: the row's address is wave-uniform (scalar base, one lane offset)
    if (L == LEV_WAVE) row_c = (uint32_t)__builtin_amdgcn_readfirstlane((int)row_c);
#pragma unroll
    for (int p = 0; p < P; ++p) {
        uint32_t g = lu + p * L;
        const bool ok = row < rows && g < units;
        q6_load_unit(w + row_c * row_bytes, g < units ? g : units - 1u, W[p]);
        W[p].d = ok ? W[p].d : 0u;
    }
}

// L lanes per row-part, P passes of L units, S waves share a row (units <=
// S*L*P; S > 1 only with L = 64 and P = 1).  RESIDENT: the lane keeps the digit
// planes of its P units in registers for every row; otherwise (rows wider than
// 128 units) it reads them from LDS per row.
// S = 2 is the shape of a 4096-wide row: one unit per lane keeps the kernel
// under 100 registers, five waves per SIMD, which is what both the vector ALU
// (a single wave issues one instruction every 8 cycles, the SIMD takes one
// every 2) and the memory latency need; the two waves of a row meet in LDS, one
// barrier per tile (two buffers).
// Persistent workgroups of four waves, the next tile's weights in flight while
// the current one is multiplied.
// partials (optional): the workgroup's top two logits and the index of the
// best, one float4 {best, second, idx bits, 0} per workgroup, for the greedy
// token epilogue.
template <int L, int P, bool RESIDENT, int S>
__global__ void __launch_bounds__(kThreads)
q6_k_gemv_exact(const uint8_t *__restrict__ w, const float *__restrict__ x, float *__restrict__ y,
                uint32_t units, uint32_t rows, lev_f32x4 *__restrict__ partials) {
    extern __shared__ lev_u32x4 xs[];
    static_assert(S == 1 || (L == LEV_WAVE && P == 1), "rows are shared by whole waves only");
    constexpr int G = LEV_WAVE / L;
    constexpr uint32_t kRowsPerTile = kWaves * G / S;
    __shared__ double part[2][S > 1 ? kWaves : 1];
    q6_group_meta *meta = reinterpret_cast<q6_group_meta *>(xs + 8u * (units + 1u));
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
    constexpr int kDepth = (P == 1) ? LEV_Q6_DEPTH : 2;
    q6_unit_w W[kDepth][P];
    q6_load_row<L, P>(w, row_bytes, base + in_tile, rows, lu, units, W[0]);
    const bool finite = q6_stage_digits(x, xs, meta, units, tid);   // ends with a barrier

    constexpr int PR = RESIDENT ? P : 1;
    q6_unit_xi X[PR];
    q6_group_meta Mlo[PR], Mhi[PR];
    if (RESIDENT) {
#pragma unroll
        for (int p = 0; p < P; ++p) {
            const uint32_t g = lu + p * L;
            q6_fetch_digits(xs, meta, units, g < units ? g : units - 1u, X[p], Mlo[p], Mhi[p]);
        }
    }
    const float poison = finite ? 0.f : __builtin_nanf("");   // a NaN or infinity in x reaches every output
    auto note = [&](float out, uint32_t row) {
        // running top two of the rows this lane finishes (rows ascend, so a
        // tie keeps the earlier, lower index)
        if (out > m.best) {
            m.second = m.best;
            m.best = out;
            m.idx = row;
        } else if (out > m.second) {
            m.second = out;
        }
    };

    uint32_t buf = 0;
    auto finish = [&](uint32_t row, const q6_unit_w (&W)[P]) {
        double acc = 0.0;
#pragma unroll
        for (int p = 0; p < P; ++p) {
            const uint32_t g = lu + p * L;
            if (RESIDENT) {
                acc += q6_unit_dot_exact(W[p], X[p], Mlo[p], Mhi[p], g & 3u);
            } else {
                q6_fetch_digits(xs, meta, units, g < units ? g : units - 1u, X[0], Mlo[0], Mhi[0]);
                acc += q6_unit_dot_exact(W[p], X[0], Mlo[0], Mhi[0], g & 3u);
            }
        }
        acc = lev_group_sum_f64<L>(acc);
        if constexpr (S == 1) {
            if (lane % L == L - 1 && row < rows) {
                const float out = (float)acc + poison;
                y[row] = out;
                note(out, row);
            }
        } else {
            // the odd wave of a row leaves its half in LDS, the even one adds and stores
            if ((wave & 1u) && lane == LEV_WAVE - 1) part[buf][wave >> 1] = acc;
            lev_barrier_lds();   // not __syncthreads(): the next tiles' loads stay in flight
            if (!(wave & 1u) && lane == LEV_WAVE - 1 && row < rows) {
                const float out = (float)(acc + part[buf][wave >> 1]) + poison;
                y[row] = out;
                note(out, row);
            }
            buf ^= 1u;
        }
    };
    // kDepth tiles in flight per wave (the one being multiplied and kDepth-1
    // behind it): what the streaming rate of this kernel is made of is bytes in
    // flight over memory latency.  The prefetch is unconditional (clamped past
    // the end): a branch around the loads would make the compiler wait for them
    // before the current row is used.
#pragma unroll
    for (int k = 1; k < kDepth - 1; ++k)
        q6_load_row<L, P>(w, row_bytes, base + k * step + in_tile, rows, lu, units, W[k]);
    for (bool more = true; more;) {
#pragma unroll
        for (int k = 0; k < kDepth; ++k) {
            q6_load_row<L, P>(w, row_bytes, base + (kDepth - 1) * step + in_tile, rows, lu, units,
                              W[(k + kDepth - 1) % kDepth]);
            finish(base + in_tile, W[k]);
            base += step;
            if (base >= rows) {   // uniform over the workgroup
                more = false;
                break;
            }
        }
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

// One workgroup: merges the per-workgroup partials of the GEMV (n <= 4096).
// All of a thread's partials are requested before the first is used: one
// memory round trip, not one per partial.
__global__ void __launch_bounds__(1024)
argmax_partials_kernel(const lev_f32x4 *__restrict__ partials, uint32_t n,
                       uint32_t *__restrict__ out_idx, float *__restrict__ out_margin) {
    __shared__ float s_best[16], s_second[16];
    __shared__ uint32_t s_idx[16];
    const uint32_t t = threadIdx.x;
    lev_f32x4 p[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const uint32_t i = t + 1024u * (uint32_t)k;
        p[k] = partials[i < n ? i : n - 1u];
    }
    top2 m{kTop2Floor, kTop2Floor, 0xFFFFFFFFu};
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const float idx_bits = p[k].z;   // a copy: bit_cast straight from a vector element reads element 0
        if (t + 1024u * (uint32_t)k < n) m = top2_merge(m, top2{p[k].x, p[k].y, __float_as_uint(idx_bits)});
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
        for (int k = 1; k < 16; ++k) r = top2_merge(r, top2{s_best[k], s_second[k], s_idx[k]});
        if (out_idx) out_idx[0] = r.idx == 0xFFFFFFFFu ? 0u : r.idx;   // nothing above -inf: first
        if (out_margin) out_margin[0] = r.best - r.second;
    }
}

// Any in_dim and alignment: one wave per row, activations read through the
// cache, 16-element sums in f32 (two chains), everything behind them in f64.
__global__ void __launch_bounds__(kThreads)
q6_k_gemv_generic(const uint8_t *__restrict__ w, const float *__restrict__ x,
                  float *__restrict__ y, uint32_t units, uint32_t rows) {
    const uint32_t lane = threadIdx.x & (LEV_WAVE - 1);
    const uint32_t row = blockIdx.x * kWaves + threadIdx.x / LEV_WAVE;
    if (row >= rows) return;
    const uint8_t *rp = w + (uint64_t)row * (units >> 3) * 210u;
    double acc = 0.0;
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
    acc = lev_group_sum_f64<64>(acc);
    if (lane == LEV_WAVE - 1) y[row] = (float)acc;
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

template <int L, int P, bool RESIDENT = true, int S = 1>
hipError_t launch_units(lev_ctx *ctx, const uint8_t *w, const float *x, float *y, uint32_t units,
                        uint32_t rows, uint32_t *d_argmax, float *d_margin) {
    constexpr uint32_t rows_per_tile = kWaves * (LEV_WAVE / L) / S;
    uint32_t blocks = (rows + rows_per_tile - 1) / rows_per_tile;
    const size_t lds = q6_lds_bytes(units);
    // persistent grid: exactly the workgroups that are resident at once, so
    // that no workgroup waits for a slot behind another one's whole loop
    int per_cu = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, q6_k_gemv_exact<L, P, RESIDENT, S>, kThreads, lds) !=
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
    hipLaunchKernelGGL((q6_k_gemv_exact<L, P, RESIDENT, S>), dim3(blocks), dim3(kThreads), lds, ctx->stream, w,
                       x, y, units, rows, partials);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess || !partials) return e;
    hipLaunchKernelGGL(argmax_partials_kernel, dim3(1), dim3(1024), 0, ctx->stream, partials, blocks,
                       d_argmax, d_margin);
    return hipGetLastError();
}

}  // namespace

uint32_t lev_q6_k_mfma_cols(const lev_ctx *ctx, uint32_t in_dim);
uint32_t lev_q6_k_mfma_waves(const lev_ctx *ctx, uint32_t in_dim, uint32_t rows);
hipError_t lev_q6_k_mfma_gemv_launch(lev_ctx *ctx, const uint8_t *w, const float *x, const float *gain,
                                     float eps, float *y, uint32_t in_dim, uint32_t rows, uint32_t ncol,
                                     uint32_t waves, lev_f32x4 *partials, uint32_t *d_argmax, float *d_margin);

namespace {
bool q6_mfma_usable(const lev_ctx *ctx, const uint8_t *w, const float *x, uint32_t in_dim) {
    return ((reinterpret_cast<uintptr_t>(w) & 1u) == 0u) && ((reinterpret_cast<uintptr_t>(x) & 15u) == 0u) &&
           lev_q6_k_mfma_cols(ctx, in_dim) >= 1u;
}

bool q6_exact_usable(const uint8_t *w, const float *x, uint32_t units) {
    return ((reinterpret_cast<uintptr_t>(w) & 1u) == 0u) && ((reinterpret_cast<uintptr_t>(x) & 15u) == 0u) &&
           units <= 256u;
}
}  // namespace

// Candidate schedules of a Q6_K GEMV shape, the built-in choice first (vk_q6k,
// lev-cli/src/main.rs:467; the q6k.matvec variants of lev-forge/src/q6k.rs:175):
// the integer matrix-core kernel (family 2; rows_in_flight = waves per row group: the
// built-in count, then 2 and 4 where they differ), the digit-plane dot4 kernel (family
// 0), for rows of 65..128 units with two waves or one wave per row, and the
// one-wave-per-row kernel with f64 sums (family 1).  (Pointer alignment
// is not part of a shape: a selection of the exact kernel is ignored for operands
// it cannot take.)
uint32_t lev_q6_k_gemv_candidates(const lev_ctx *ctx, uint32_t in_dim, uint32_t rows, lev_schedule *out,
                                  uint32_t capacity) {
    const uint32_t units = in_dim / 32u;
    uint32_t n = 0;
    auto add = [&](uint32_t family, uint32_t waves) {
        if (n < capacity) out[n] = lev_schedule{LEV_OP_Q6_K_GEMV, family, waves, 0u};
        ++n;
    };
    if (lev_q6_k_mfma_cols(ctx, in_dim) >= 1u) {
        // rows of at most sixteen superblocks: a wave per superblock column (schedule field 0 waves
        // per row group), the built-in choice there; then the several-column kernel at one column
        if (in_dim <= 4096u) add(2u, 0u);
        const uint32_t builtin = lev_q6_k_mfma_waves(ctx, in_dim, rows);
        add(2u, builtin);
        if (builtin != 2u) add(2u, 2u);
        if (builtin != 4u) add(2u, 4u);
    }
    if (units <= 256u) {
        const bool pair = units > 64u && units <= 128u;
        add(0u, pair ? 2u : 1u);
        if (pair) add(0u, 1u);
    }
    add(1u, 1u);
    return n;
}

// GEMV with the greedy-token epilogue: d_argmax / d_margin may be NULL.
hipError_t lev_q6_k_gemv_argmax_launch(lev_ctx *ctx, const uint8_t *w, const float *x, float *y,
                                       uint32_t in_dim, uint32_t rows, uint32_t *d_argmax,
                                       float *d_margin) {
    const uint32_t units = in_dim / 32u;   // 8 per superblock
    // a schedule installed for this shape (lev_hip_forge_select) overrides the built-in choice
    const lev_schedule *sel = lev_selected(ctx, LEV_OP_Q6_K_GEMV, in_dim, rows, 1);
    const uint32_t family = sel ? sel->family : 2u;
    if (family == 2u && q6_mfma_usable(ctx, w, x, in_dim)) {
        return lev_q6_k_mfma_gemv_launch(ctx, w, x, nullptr, 0.f, y, in_dim, rows, 1,
                                         sel ? sel->rows_in_flight : 0u,
                                         static_cast<lev_f32x4 *>(ctx->argmax_partials), d_argmax, d_margin);
    }
    const bool fast = q6_exact_usable(w, x, units) && family != 1u;
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
    if (units > 128) return launch_units<64, 4, false>(ctx, w, x, y, units, rows, d_argmax, d_margin);
    if (units > 64) {
        if (sel && sel->rows_in_flight == 1u)
            return launch_units<64, 2, true, 1>(ctx, w, x, y, units, rows, d_argmax, d_margin);
        return launch_units<64, 1, true, 2>(ctx, w, x, y, units, rows, d_argmax, d_margin);
    }
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

extern "C" int lev_hip_q6_k_gemv_ncol(lev_ctx *ctx, const void *d_w, size_t w_bytes, uint64_t w_off,
                                      const float *d_x, size_t x_count, const float *d_gain,
                                      float eps, float *d_y, size_t y_capacity, uint32_t in_dim,
                                      uint32_t rows, uint32_t ncol) {
    LEV_REQUIRE_CTX(ctx);
    if (ncol == 0 || ncol > LEV_MAX_GEMV_COLUMNS)
        return lev_fail(ctx, LEV_ERR_BAD_DIMENSIONS, "q6_k_gemv_ncol: %u columns (1..%d)", ncol,
                        LEV_MAX_GEMV_COLUMNS);
    if (d_gain && !(eps >= 0.f))
        return lev_fail(ctx, LEV_ERR_BAD_DIMENSIONS, "q6_k_gemv_ncol: eps %g", (double)eps);
    lev_geom g;
    int st = lev_check_matvec(ctx, "q6_k_gemv_ncol", 256, 210, d_w, w_bytes, w_off, d_x, x_count,
                              (uint64_t)in_dim * ncol, d_y, y_capacity, (uint64_t)rows * ncol,
                              in_dim, rows, &g);
    if (st != LEV_OK) return st;
    const uint8_t *w = static_cast<const uint8_t *>(d_w) + w_off;
    if ((reinterpret_cast<uintptr_t>(w) & 1u) || (reinterpret_cast<uintptr_t>(d_x) & 15u) ||
        (d_gain && (reinterpret_cast<uintptr_t>(d_gain) & 15u)))
        return lev_fail(ctx, LEV_ERR_BAD_DIMENSIONS,
                        "q6_k_gemv_ncol: weights must be 2-byte, x and gain 16-byte aligned");
    const uint32_t per_launch = lev_q6_k_mfma_cols(ctx, in_dim);
    if (per_launch == 0)
        return lev_fail(ctx, LEV_ERR_EXCEEDS_MODEL_WORKLOAD,
                        "q6_k_gemv_ncol: inDim %u does not fit the activation staging", in_dim);
    for (uint32_t c0 = 0; c0 < ncol; c0 += per_launch) {
        const uint32_t nc = ncol - c0 < per_launch ? ncol - c0 : per_launch;
        st = lev_hip_check(ctx,
                           lev_q6_k_mfma_gemv_launch(ctx, w, d_x + (uint64_t)c0 * in_dim, d_gain, eps,
                                                     d_y + (uint64_t)c0 * rows, in_dim, rows, nc, 0u, nullptr,
                                                     nullptr, nullptr),
                           "q6_k_gemv_ncol launch");
        if (st != LEV_OK) return st;
    }
    return LEV_OK;
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

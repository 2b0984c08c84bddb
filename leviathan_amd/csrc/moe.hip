// MoE layer for gfx950: router + softmax/top-k, routed Q4_0 experts
// (gate/up + GELU*up fused, down + ordered weighted merge).
//
// Stands in for the MoE block of forwardLayer (Gemma4.swift:3795-3880):
//   g4_f32_matvec (:4160) + CPU softmax/top-k (:3801-3810),
//   runMoeBatchedRouted (:2073) with moegen_gu/act/dn (MoELowering.swift:749-835)
//   or the fused moesimd_gu / moesimd_dn (MoESIMDLowering.swift:497-636),
//   and the ordered g4_axpy merges (:2171-2175, :4459).
//
// Three launches per call, all HBM-bound:
//   1. router: one wave per (token, expert) row, f64 accumulation; the last
//      wave to finish a token runs softmax (f64), top-k (ties -> lower index)
//      and renormalisation for that token.
//   2. gate/up: a wave streams gate row i with lanes 0..31 and up row i with
//      lanes 32..63 (a row of 2048 values is 32 block pairs), reduces both and
//      writes act = gelu_tanh(g)*u.  x is staged once per workgroup.
//   3. down: wave s of a workgroup streams the rows of slot s for the
//      workgroup's tile of outputs; partial results meet in LDS and are merged
//      IN SLOT ORDER in f32, as the reference's axpy chain does.
#include "q4_0_device.hpp"

namespace {

constexpr int kFlagBadExpertId = 1;
constexpr int kFlagNonFiniteScore = 2;

// ---------------------------------------------------------------------------
// router
// ---------------------------------------------------------------------------

__device__ __forceinline__ double wave_sum_f64(double v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
    return v;
}

// grid (experts, tokens), 64 threads.  counters[tokens] must be zero on entry
// and are zero again on exit (atomicInc wraps at experts-1).
__global__ void __launch_bounds__(64)
moe_router_kernel(const float *__restrict__ wr, const float *__restrict__ x,
                  const float *__restrict__ expert_scale, float *__restrict__ scores,
                  int32_t *__restrict__ ids, float *__restrict__ weights,
                  uint32_t *__restrict__ counters, int *__restrict__ flag, uint32_t hidden,
                  uint32_t experts, uint32_t top_k) {
    const uint32_t e = blockIdx.x, t = blockIdx.y, lane = threadIdx.x;
    const float *row = wr + (uint64_t)e * hidden;
    const float *xv = x + (uint64_t)t * hidden;
    double acc = 0.0;
    if ((hidden & 3u) == 0u) {
        const lev_f32x4 *r4 = reinterpret_cast<const lev_f32x4 *>(row);
        const lev_f32x4 *x4 = reinterpret_cast<const lev_f32x4 *>(xv);
        double a0 = 0.0, a1 = 0.0;
        for (uint32_t i = lane; i < hidden / 4u; i += 64u) {
            lev_f32x4 a = r4[i], b = x4[i];
            a0 = fma((double)a.x, (double)b.x, a0);
            a1 = fma((double)a.y, (double)b.y, a1);
            a0 = fma((double)a.z, (double)b.z, a0);
            a1 = fma((double)a.w, (double)b.w, a1);
        }
        acc = a0 + a1;
    } else {
        for (uint32_t i = lane; i < hidden; i += 64u) acc = fma((double)row[i], (double)xv[i], acc);
    }
    acc = wave_sum_f64(acc);
    float *srow = scores + (uint64_t)t * experts;
    uint32_t done = 0;
    if (lane == 0) {
        __hip_atomic_store(&srow[e], (float)acc, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __threadfence();
        done = atomicInc(&counters[t], experts - 1u);
    }
    done = __shfl(done, 0);
    if (done != experts - 1u) return;
    __threadfence();

    // ---- last wave of this token: softmax + top-k (Gemma4.swift:3798-3810) ----
    extern __shared__ double s_p[];                 // experts doubles
    float mx = -INFINITY;
    bool finite = true;
    for (uint32_t i = lane; i < experts; i += 64u) {
        float s = __hip_atomic_load(&srow[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        finite = finite && isfinite(s);
        mx = fmaxf(mx, s);
        s_p[i] = (double)s;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
    if (__any(!finite)) {
        if (lane == 0) atomicOr(flag, kFlagNonFiniteScore);
        for (uint32_t k = lane; k < top_k; k += 64u) {
            ids[(uint64_t)t * top_k + k] = (int32_t)k;
            weights[(uint64_t)t * top_k + k] = 0.f;
        }
        return;
    }
    double sum = 0.0;
    for (uint32_t i = lane; i < experts; i += 64u) {
        double p = exp((double)((float)s_p[i] - mx));   // subtraction in f32, exp in f64
        s_p[i] = p;
        sum += p;
    }
    sum = wave_sum_f64(sum);
    for (uint32_t i = lane; i < experts; i += 64u) s_p[i] = s_p[i] / sum;
    __builtin_amdgcn_s_barrier();   // single wave: orders the LDS writes above
    double prob_sum = 0.0;
    double my_p = 0.0;              // lane k keeps the probability of slot k (top_k <= 64)
    uint32_t my_id = 0;
    for (uint32_t k = 0; k < top_k; ++k) {
        double best = -1.0;
        uint32_t bi = 0xFFFFFFFFu;
        for (uint32_t i = lane; i < experts; i += 64u) {
            double p = s_p[i];
            if (p > best) {       // ascending i within a lane: ties keep the lower index
                best = p;
                bi = i;
            }
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            double ob = __shfl_xor(best, off);
            uint32_t oi = __shfl_xor(bi, off);
            if (ob > best || (ob == best && oi < bi)) {
                best = ob;
                bi = oi;
            }
        }
        prob_sum += best;          // slot order, as topIdx.reduce does
        if (lane == k) {
            my_p = best;
            my_id = bi;
        }
        if (lane == (bi & 63u)) s_p[bi] = -2.0;   // taken
        __builtin_amdgcn_s_barrier();
    }
    if (lane < top_k) {
        float wgt = (float)(my_p / prob_sum);
        if (expert_scale) wgt *= expert_scale[my_id];
        ids[(uint64_t)t * top_k + lane] = (int32_t)my_id;
        weights[(uint64_t)t * top_k + lane] = wgt;
    }
}

// ---------------------------------------------------------------------------
// expert ids: bounds + distinctness (MoEModelBinding.offsets requires both)
// ---------------------------------------------------------------------------

__device__ __forceinline__ bool expert_ids_ok(const int32_t *ids, uint32_t top_k, uint32_t slot,
                                              uint32_t experts) {
    int32_t me = ids[slot];
    if (me < 0 || (uint32_t)me >= experts) return false;
    for (uint32_t k = 0; k < top_k; ++k)
        if (k != slot && ids[k] == me) return false;
    return true;
}

// ---------------------------------------------------------------------------
// gate/up + GELU*up
// ---------------------------------------------------------------------------

struct moe_args {
    const uint8_t *base;
    uint64_t gate_off, up_off, down_off;
    uint64_t gate_stride, up_stride, down_stride;
    uint32_t hidden, inter, experts, top_k;
};

constexpr int kGuThreads = 256;
constexpr int kGuWaves = kGuThreads / LEV_WAVE;

// grid (chunks_per_slot, top_k, tokens).  P = passes of 32 pairs per row.
template <int P>
__global__ void __launch_bounds__(kGuThreads)
moe_gate_up_kernel(moe_args a, const float *__restrict__ x, const int32_t *__restrict__ ids,
                   float *__restrict__ act, int *__restrict__ flag, uint32_t rows_per_block) {
    extern __shared__ lev_f32x4 xs[];
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t slot = blockIdx.y, t = blockIdx.z;
    const uint32_t pairs = a.hidden / 64u;
    const uint32_t half = lane >> 5, lp = lane & 31u;
    const int32_t *tids = ids + (uint64_t)t * a.top_k;
    if (!expert_ids_ok(tids, a.top_k, slot, a.experts)) {
        if (tid == 0) atomicOr(flag, kFlagBadExpertId);
        return;
    }
    const uint32_t e = (uint32_t)tids[slot];
    const uint64_t row_bytes = (uint64_t)pairs * 36u;
    // lanes 0..31 walk the gate row, lanes 32..63 the up row of the same index
    const uint8_t *wbase = a.base + (half ? a.up_off + e * a.up_stride : a.gate_off + e * a.gate_stride);
    const uint32_t i_begin = blockIdx.x * rows_per_block;
    const uint32_t i_end = min(i_begin + rows_per_block, a.inter);

    lev_f32x4 xv[kLevStageSlots];
    const float *xt = x + (uint64_t)t * a.hidden;
    lev_q4_stage_x_load(xt, pairs, tid, kGuThreads, xv);

    uint32_t Da[P][9], Db[P][9];
    auto load_row = [&](uint32_t i, uint32_t (&D)[P][9]) {
        const uint8_t *rp = wbase + (uint64_t)(i < i_end ? i : i_end - 1u) * row_bytes;
#pragma unroll
        for (int p = 0; p < P; ++p) {
            uint32_t pr = lp + 32u * p;
            lev_q4_load_pair(rp + (uint64_t)(pr < pairs ? pr : pairs - 1u) * 36u, D[p]);
        }
    };
    uint32_t i = i_begin + wave;
    load_row(i, Da);
    lev_q4_stage_x_store(xt, xs, pairs, tid, kGuThreads, xv);
    __syncthreads();
    if (i >= i_end) return;

    lev_q4_pair_x X[P];
#pragma unroll
    for (int p = 0; p < P; ++p) {
        uint32_t pr = lp + 32u * p;
        lev_q4_fetch_x(xs, pairs, pr < pairs ? pr : pairs - 1u, X[p]);
        if (pr >= pairs) {   // padding lanes contribute nothing
#pragma unroll
            for (int q = 0; q < 16; ++q) X[p].xr[q] = lev_f32x4{0.f, 0.f, 0.f, 0.f};
            X[p].sum_a = X[p].sum_b = 0.f;
        }
    }
    float *arow = act + ((uint64_t)t * a.top_k + slot) * a.inter;
    auto finish_row = [&](uint32_t i, const uint32_t (&D)[P][9]) {
        float acc = 0.f;
#pragma unroll
        for (int p = 0; p < P; ++p) acc += lev_q4_pair_dot(D[p], X[p]);
        acc = lev_group_sum<32>(acc);
        float g = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, acc), 31));
        float u = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, acc), 63));
        if (lane == 0) arow[i] = lev_gelu_up_value(g, u);
    };
    while (true) {
        uint32_t next = i + kGuWaves;
        if (next < i_end) load_row(next, Db);
        finish_row(i, Da);
        if (next >= i_end) break;
        i = next;
        next = i + kGuWaves;
        if (next < i_end) load_row(next, Da);
        finish_row(i, Db);
        if (next >= i_end) break;
        i = next;
    }
}

// ---------------------------------------------------------------------------
// down + ordered merge
// ---------------------------------------------------------------------------

constexpr int kDnWaves = 8;
constexpr int kDnThreads = kDnWaves * LEV_WAVE;

// grid (row_tiles, tokens).  L lanes per row (pairs <= L), G = 64/L rows per
// wave-step, `steps` wave-steps per tile: tile = G*steps rows.
// LDS: per wave a transposed copy of its slot's activations, then
// top_k*tile partial sums.
template <int L>
__global__ void __launch_bounds__(kDnThreads)
moe_down_kernel(moe_args a, const float *__restrict__ act, const int32_t *__restrict__ ids,
                const float *__restrict__ weights, float *__restrict__ y, int *__restrict__ flag,
                uint32_t steps) {
    extern __shared__ lev_f32x4 lds[];
    constexpr uint32_t G = LEV_WAVE / L;
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t t = blockIdx.y;
    const uint32_t pairs = a.inter / 64u;
    const uint32_t tile = G * steps;
    const uint32_t row_begin = blockIdx.x * tile;
    const uint32_t grp = lane / L, lp = lane % L;
    const uint64_t row_bytes = (uint64_t)pairs * 36u;
    const uint32_t x_slots = 16u * (pairs + 1u);
    lev_f32x4 *xs = lds + wave * x_slots;
    float *partial = reinterpret_cast<float *>(lds + kDnWaves * x_slots);   // [top_k][tile]
    const int32_t *tids = ids + (uint64_t)t * a.top_k;
    const uint32_t pc = lp < pairs ? lp : pairs - 1u;

    bool bad = false;
    for (uint32_t slot = wave; slot < a.top_k; slot += kDnWaves) {
        if (!expert_ids_ok(tids, a.top_k, slot, a.experts)) {
            bad = true;
            for (uint32_t r = lane; r < tile; r += 64u) partial[slot * tile + r] = 0.f;
            continue;
        }
        const uint32_t e = (uint32_t)tids[slot];
        const uint8_t *wbase = a.base + a.down_off + e * a.down_stride;
        // first rows' weights go out before the activations are touched
        uint32_t Da[9], Db[9];
        auto load_row = [&](uint32_t step, uint32_t (&D)[9]) {
            uint32_t row = row_begin + step * G + grp;
            lev_q4_load_pair(wbase + (uint64_t)(row < a.hidden ? row : a.hidden - 1u) * row_bytes +
                                 (uint64_t)pc * 36u, D);
        };
        load_row(0, Da);
        // this wave's slot activations -> its private LDS region (wave-local)
        const float *av = act + ((uint64_t)t * a.top_k + slot) * a.inter;
        lev_q4_stage_x(av, xs, pairs, lane, 64u);
        // wave-private region: LDS executes one wave's accesses in order, the
        // fences only stop the compiler from moving the reads above the writes
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        lev_q4_pair_x X;
        lev_q4_fetch_x(xs, pairs, pc, X);
        if (lp >= pairs) {
#pragma unroll
            for (int q = 0; q < 16; ++q) X.xr[q] = lev_f32x4{0.f, 0.f, 0.f, 0.f};
            X.sum_a = X.sum_b = 0.f;
        }
        auto finish_row = [&](uint32_t step, const uint32_t (&D)[9]) {
            float s = lev_group_sum<L>(lev_q4_pair_dot(D, X));
            if (lp == L - 1) partial[slot * tile + step * G + grp] = s;
        };
        uint32_t step = 0;
        while (true) {
            if (step + 1 < steps) load_row(step + 1, Db);
            finish_row(step, Da);
            if (++step >= steps) break;
            if (step + 1 < steps) load_row(step + 1, Da);
            finish_row(step, Db);
            if (++step >= steps) break;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();   // X reads done before the next slot restages xs
    }
    if (bad && lane == 0) atomicOr(flag, kFlagBadExpertId);
    __syncthreads();
    // ordered merge: y = sum over slots, in slot order, of w_slot * dn[slot]
    for (uint32_t r = tid; r < tile; r += kDnThreads) {
        uint32_t row = row_begin + r;
        if (row >= a.hidden) continue;
        float accum = 0.f;
        for (uint32_t slot = 0; slot < a.top_k; ++slot)
            accum = fmaf(weights[(uint64_t)t * a.top_k + slot], partial[slot * tile + r], accum);
        y[(uint64_t)t * a.hidden + row] = accum;
    }
}

// ---------------------------------------------------------------------------
// generic expert path (odd block counts, unaligned pools, very long rows):
// one wave per output row, 16-bit loads, activations through the cache.
// ---------------------------------------------------------------------------

__device__ __forceinline__ float q4_0_row_dot_generic(const uint8_t *rp, const float *x,
                                                      uint32_t blocks, uint32_t lane) {
    float acc = 0.f;
    for (uint32_t b = lane; b < blocks; b += LEV_WAVE) {
        const uint16_t *h = reinterpret_cast<const uint16_t *>(rp + (uint64_t)b * 18u);
        float d = lev_f16_bits_to_f32(h[0]);
        const float *xb = x + (uint64_t)b * 32u;
        float s = 0.f, xsum = 0.f;
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            uint32_t two = h[1 + k];
            float x0 = xb[2 * k], x1 = xb[2 * k + 1], x2 = xb[16 + 2 * k], x3 = xb[17 + 2 * k];
            s = fmaf((float)(two & 0xF), x0, s);
            s = fmaf((float)((two >> 8) & 0xF), x1, s);
            s = fmaf((float)((two >> 4) & 0xF), x2, s);
            s = fmaf((float)(two >> 12), x3, s);
            xsum += (x0 + x1) + (x2 + x3);
        }
        acc = fmaf(d, fmaf(-8.0f, xsum, s), acc);
    }
    acc = lev_group_sum<64>(acc);
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, acc), 63));
}

// grid (ceil(inter/4), top_k, tokens), 256 threads
__global__ void __launch_bounds__(256)
moe_gate_up_generic(moe_args a, const float *__restrict__ x, const int32_t *__restrict__ ids,
                    float *__restrict__ act, int *__restrict__ flag) {
    const uint32_t lane = threadIdx.x & 63u, i = blockIdx.x * 4u + (threadIdx.x >> 6);
    const uint32_t slot = blockIdx.y, t = blockIdx.z;
    const int32_t *tids = ids + (uint64_t)t * a.top_k;
    if (!expert_ids_ok(tids, a.top_k, slot, a.experts)) {
        if (threadIdx.x == 0) atomicOr(flag, kFlagBadExpertId);
        return;
    }
    if (i >= a.inter) return;
    const uint32_t e = (uint32_t)tids[slot], blocks = a.hidden / 32u;
    const float *xt = x + (uint64_t)t * a.hidden;
    float g = q4_0_row_dot_generic(a.base + a.gate_off + e * a.gate_stride + (uint64_t)i * blocks * 18u,
                                   xt, blocks, lane);
    float u = q4_0_row_dot_generic(a.base + a.up_off + e * a.up_stride + (uint64_t)i * blocks * 18u,
                                   xt, blocks, lane);
    if (lane == 0) act[((uint64_t)t * a.top_k + slot) * a.inter + i] = lev_gelu_up_value(g, u);
}

// grid (ceil(hidden/4), tokens), 256 threads: a wave owns one output row and
// walks the slots in order.
__global__ void __launch_bounds__(256)
moe_down_generic(moe_args a, const float *__restrict__ act, const int32_t *__restrict__ ids,
                 const float *__restrict__ weights, float *__restrict__ y, int *__restrict__ flag) {
    const uint32_t lane = threadIdx.x & 63u, row = blockIdx.x * 4u + (threadIdx.x >> 6);
    const uint32_t t = blockIdx.y;
    if (row >= a.hidden) return;
    const int32_t *tids = ids + (uint64_t)t * a.top_k;
    const uint32_t blocks = a.inter / 32u;
    float accum = 0.f;
    for (uint32_t slot = 0; slot < a.top_k; ++slot) {
        if (!expert_ids_ok(tids, a.top_k, slot, a.experts)) {
            if (lane == 0) atomicOr(flag, kFlagBadExpertId);
            continue;
        }
        const uint32_t e = (uint32_t)tids[slot];
        float d = q4_0_row_dot_generic(
            a.base + a.down_off + e * a.down_stride + (uint64_t)row * blocks * 18u,
            act + ((uint64_t)t * a.top_k + slot) * a.inter, blocks, lane);
        accum = fmaf(weights[(uint64_t)t * a.top_k + slot], d, accum);
    }
    if (lane == 0) y[(uint64_t)t * a.hidden + row] = accum;
}

template <int P>
hipError_t launch_gate_up(lev_ctx *ctx, const moe_args &a, const float *x, const int32_t *ids,
                          float *act, uint32_t tokens) {
    // rows per workgroup: enough workgroups to cover every CU a few times at
    // one token, more rows per workgroup (less re-staging of x) at many.
    uint64_t slots = (uint64_t)a.top_k * tokens;
    uint32_t want_blocks_per_slot = (uint32_t)(((uint64_t)ctx->num_cus * 4u + slots - 1) / slots);
    if (want_blocks_per_slot < 1) want_blocks_per_slot = 1;
    uint32_t rows_per_block = (a.inter + want_blocks_per_slot - 1) / want_blocks_per_slot;
    if (rows_per_block < (uint32_t)kGuWaves * 2u) rows_per_block = kGuWaves * 2u;
    rows_per_block = (rows_per_block + kGuWaves - 1) / kGuWaves * kGuWaves;
    uint32_t chunks = (a.inter + rows_per_block - 1) / rows_per_block;
    size_t lds = (size_t)16 * (a.hidden / 64u + 1u) * sizeof(lev_f32x4);
    hipLaunchKernelGGL((moe_gate_up_kernel<P>), dim3(chunks, a.top_k, tokens), dim3(kGuThreads), lds,
                       ctx->stream, a, x, ids, act, ctx->d_flag, rows_per_block);
    return hipGetLastError();
}

template <int L>
hipError_t launch_down(lev_ctx *ctx, const moe_args &a, const float *act, const int32_t *ids,
                       const float *weights, float *y, uint32_t tokens) {
    constexpr uint32_t G = LEV_WAVE / L;
    // tile rows: aim at >= 2 workgroups per CU at one token
    uint32_t want_tiles = (uint32_t)(((uint64_t)ctx->num_cus * 2u + tokens - 1) / tokens);
    if (want_tiles < 1) want_tiles = 1;
    uint32_t tile = (a.hidden + want_tiles - 1) / want_tiles;
    uint32_t steps = (tile + G - 1) / G;
    if (steps < 2) steps = 2;
    if (steps > 64) steps = 64;
    tile = steps * G;
    uint32_t tiles = (a.hidden + tile - 1) / tile;
    size_t lds = (size_t)kDnWaves * 16 * (a.inter / 64u + 1u) * sizeof(lev_f32x4) +
                 (size_t)a.top_k * tile * sizeof(float);
    if (lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&moe_down_kernel<L>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL((moe_down_kernel<L>), dim3(tiles, tokens), dim3(kDnThreads), lds, ctx->stream,
                       a, act, ids, weights, y, ctx->d_flag, steps);
    return hipGetLastError();
}

int check_pools(lev_ctx *ctx, const lev_moe_experts *p, uint32_t top_k, uint32_t tokens,
                moe_args *out) {
    if (!p || !p->d_base) return lev_fail(ctx, LEV_ERR_INVALID_ARGUMENT, "moe: null pools");
    if (p->hidden == 0 || p->inter == 0 || p->experts == 0 || p->hidden % 32u || p->inter % 32u ||
        p->hidden > LEV_MAX_Q4_INPUT_DIM || p->inter > LEV_MAX_Q4_INPUT_DIM)
        return lev_fail(ctx, LEV_ERR_BAD_DIMENSIONS, "moe: hidden %u, inter %u, experts %u",
                        p->hidden, p->inter, p->experts);
    if (top_k == 0 || top_k > p->experts || top_k > 64u || tokens == 0 || tokens > 65535u)
        return lev_fail(ctx, LEV_ERR_BAD_DIMENSIONS, "moe: topK %u of %u experts, %u tokens", top_k,
                        p->experts, tokens);
    const uint64_t gu_slice = (uint64_t)p->inter * (p->hidden / 32u) * 18u;
    const uint64_t dn_slice = (uint64_t)p->hidden * (p->inter / 32u) * 18u;
    struct { uint64_t off, stride, slice; const char *name; } pools[3] = {
        {p->gate_off, p->gate_stride, gu_slice, "gate"},
        {p->up_off, p->up_stride, gu_slice, "up"},
        {p->down_off, p->down_stride, dn_slice, "down"}};
    for (auto &q : pools) {
        uint64_t span, end;
        if (__builtin_mul_overflow(q.stride, (uint64_t)(p->experts - 1), &span) ||
            __builtin_add_overflow(span, q.slice, &span) || __builtin_add_overflow(q.off, span, &end))
            return lev_fail(ctx, LEV_ERR_INTEGER_OVERFLOW, "moe: %s pool extent overflows", q.name);
        if (end > p->base_bytes)
            return lev_fail(ctx, LEV_ERR_BAD_DIMENSIONS, "moe: %s pool [%llu, %llu) beyond %zu bytes",
                            q.name, (unsigned long long)q.off, (unsigned long long)end,
                            p->base_bytes);
    }
    out->base = static_cast<const uint8_t *>(p->d_base);
    out->gate_off = p->gate_off;
    out->up_off = p->up_off;
    out->down_off = p->down_off;
    out->gate_stride = p->gate_stride;
    out->up_stride = p->up_stride;
    out->down_stride = p->down_stride;
    out->hidden = p->hidden;
    out->inter = p->inter;
    out->experts = p->experts;
    out->top_k = top_k;
    return LEV_OK;
}

bool pools_fast(const moe_args &a, const float *x) {
    auto al4 = [&](uint64_t v) { return ((reinterpret_cast<uintptr_t>(a.base) + v) & 3u) == 0; };
    return a.hidden % 64u == 0 && a.inter % 64u == 0 && a.hidden <= 8192u && a.inter <= 4096u &&
           al4(a.gate_off) && al4(a.up_off) && al4(a.down_off) && a.gate_stride % 4u == 0 &&
           a.up_stride % 4u == 0 && a.down_stride % 4u == 0 &&
           (reinterpret_cast<uintptr_t>(x) & 15u) == 0;
}

hipError_t run_experts(lev_ctx *ctx, const moe_args &a, const float *x, const int32_t *ids,
                       const float *weights, float *y, float *act, uint32_t tokens) {
    hipError_t e;
    if (!pools_fast(a, x) || (reinterpret_cast<uintptr_t>(act) & 15u)) {
        hipLaunchKernelGGL(moe_gate_up_generic, dim3((a.inter + 3) / 4, a.top_k, tokens), dim3(256), 0,
                           ctx->stream, a, x, ids, act, ctx->d_flag);
        if ((e = hipGetLastError()) != hipSuccess) return e;
        hipLaunchKernelGGL(moe_down_generic, dim3((a.hidden + 3) / 4, tokens), dim3(256), 0,
                           ctx->stream, a, act, ids, weights, y, ctx->d_flag);
        return hipGetLastError();
    }
    const uint32_t gp = a.hidden / 64u;
    if (gp <= 32) e = launch_gate_up<1>(ctx, a, x, ids, act, tokens);
    else if (gp <= 64) e = launch_gate_up<2>(ctx, a, x, ids, act, tokens);
    else if (gp <= 96) e = launch_gate_up<3>(ctx, a, x, ids, act, tokens);
    else e = launch_gate_up<4>(ctx, a, x, ids, act, tokens);
    if (e != hipSuccess) return e;
    const uint32_t dp = a.inter / 64u;
    if (dp > 32) return launch_down<64>(ctx, a, act, ids, weights, y, tokens);
    if (dp > 16) return launch_down<32>(ctx, a, act, ids, weights, y, tokens);
    if (dp > 8) return launch_down<16>(ctx, a, act, ids, weights, y, tokens);
    if (dp > 4) return launch_down<8>(ctx, a, act, ids, weights, y, tokens);
    return launch_down<4>(ctx, a, act, ids, weights, y, tokens);
}

// scratch layout: [counters u32[tokens] | scores f32[tokens*experts] | act f32[tokens*top_k*inter]]
struct moe_scratch {
    uint32_t *counters;
    float *scores;
    float *act;
};

int get_scratch(lev_ctx *ctx, uint32_t tokens, uint32_t experts, uint32_t top_k, uint32_t inter,
                moe_scratch *s) {
    // the counter region has a fixed size so that it never overlaps what an
    // earlier call with other dimensions used for scores or activations
    (void)tokens;
    size_t c_bytes = (size_t)65536 * 4;
    size_t s_bytes = ((size_t)tokens * experts * 4 + 255) & ~(size_t)255;
    size_t a_bytes = (size_t)tokens * top_k * inter * 4;
    size_t before = ctx->scratch_bytes;
    char *p = static_cast<char *>(lev_scratch(ctx, c_bytes + s_bytes + a_bytes));
    if (!p) return lev_fail(ctx, LEV_ERR_EXCEEDS_WORKING_SET, "moe: scratch allocation failed");
    if (ctx->scratch_bytes != before) {
        // fresh buffer: the router's counters must start at zero (they return
        // to zero by themselves after every launch)
        hipError_t e = lev_zero_async(ctx, p, c_bytes);
        if (e != hipSuccess) return lev_hip_check(ctx, e, "moe scratch clear");
    }
    s->counters = reinterpret_cast<uint32_t *>(p);
    s->scores = reinterpret_cast<float *>(p + c_bytes);
    s->act = reinterpret_cast<float *>(p + c_bytes + s_bytes);
    return LEV_OK;
}

hipError_t run_router(lev_ctx *ctx, const float *wr, const float *x, const float *scale,
                      float *scores, int32_t *ids, float *weights, uint32_t *counters,
                      uint32_t hidden, uint32_t experts, uint32_t top_k, uint32_t tokens) {
    hipLaunchKernelGGL(moe_router_kernel, dim3(experts, tokens), dim3(64), experts * sizeof(double),
                       ctx->stream, wr, x, scale, scores, ids, weights, counters, ctx->d_flag, hidden,
                       experts, top_k);
    return hipGetLastError();
}

}  // namespace

extern "C" int lev_hip_moe_route_topk(lev_ctx *ctx, const float *d_router_w, const float *d_x,
                                      const float *d_expert_scale, int32_t *d_ids, float *d_weights,
                                      float *d_scores, uint32_t hidden, uint32_t experts,
                                      uint32_t top_k, uint32_t tokens) {
    LEV_REQUIRE_CTX(ctx);
    if (!d_router_w || !d_x || !d_ids || !d_weights)
        return lev_fail(ctx, LEV_ERR_INVALID_ARGUMENT, "moe_route_topk: null pointer");
    if (hidden == 0 || experts == 0 || experts > 4096u || top_k == 0 || top_k > experts ||
        top_k > 64u || tokens == 0 || tokens > 65535u || hidden > LEV_MAX_Q4_INPUT_DIM)
        return lev_fail(ctx, LEV_ERR_BAD_DIMENSIONS,
                        "moe_route_topk: hidden %u, experts %u, topK %u, tokens %u", hidden, experts,
                        top_k, tokens);
    moe_scratch s;
    int st = get_scratch(ctx, tokens, experts, top_k, 0, &s);
    if (st != LEV_OK) return st;
    // With caller-provided scores the counters still live in the scratch.
    float *scores = d_scores ? d_scores : s.scores;
    return lev_hip_check(ctx,
                         run_router(ctx, d_router_w, d_x, d_expert_scale, scores, d_ids, d_weights,
                                    s.counters, hidden, experts, top_k, tokens),
                         "moe router launch");
}

extern "C" int lev_hip_moe_experts_q4_0(lev_ctx *ctx, const lev_moe_experts *pools, const float *d_x,
                                        const int32_t *d_ids, const float *d_weights, float *d_y,
                                        float *d_act, uint32_t top_k, uint32_t tokens) {
    LEV_REQUIRE_CTX(ctx);
    if (!d_x || !d_ids || !d_weights || !d_y)
        return lev_fail(ctx, LEV_ERR_INVALID_ARGUMENT, "moe_experts: null pointer");
    moe_args a;
    int st = check_pools(ctx, pools, top_k, tokens, &a);
    if (st != LEV_OK) return st;
    float *act = d_act;
    if (!act) {
        moe_scratch s;
        st = get_scratch(ctx, tokens, a.experts, top_k, a.inter, &s);
        if (st != LEV_OK) return st;
        act = s.act;
    }
    return lev_hip_check(ctx, run_experts(ctx, a, d_x, d_ids, d_weights, d_y, act, tokens),
                         "moe experts launch");
}

extern "C" int lev_hip_moe_layer_q4_0(lev_ctx *ctx, const lev_moe_experts *pools,
                                      const float *d_router_w, const float *d_expert_scale,
                                      const float *d_x, float *d_y, int32_t *d_ids, float *d_weights,
                                      uint32_t top_k, uint32_t tokens) {
    LEV_REQUIRE_CTX(ctx);
    if (!d_router_w || !d_x || !d_y || !d_ids || !d_weights)
        return lev_fail(ctx, LEV_ERR_INVALID_ARGUMENT, "moe_layer: null pointer");
    moe_args a;
    int st = check_pools(ctx, pools, top_k, tokens, &a);
    if (st != LEV_OK) return st;
    if (a.experts > 4096u) return lev_fail(ctx, LEV_ERR_BAD_DIMENSIONS, "moe_layer: %u experts", a.experts);
    moe_scratch s;
    st = get_scratch(ctx, tokens, a.experts, top_k, a.inter, &s);
    if (st != LEV_OK) return st;
    st = lev_hip_check(ctx,
                       run_router(ctx, d_router_w, d_x, d_expert_scale, s.scores, d_ids, d_weights,
                                  s.counters, a.hidden, a.experts, top_k, tokens),
                       "moe router launch");
    if (st != LEV_OK) return st;
    return lev_hip_check(ctx, run_experts(ctx, a, d_x, d_ids, d_weights, d_y, s.act, tokens),
                         "moe experts launch");
}

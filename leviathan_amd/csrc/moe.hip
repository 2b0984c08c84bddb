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
//   1. router: a workgroup per expert row, its waves take tokens in turn, f64
//      accumulation; the wave that completes a token's last score runs softmax
//      (f64), top-k (ties -> lower index) and renormalisation for that token.
//   2. gate/up: a wave streams gate row i with lanes 0..31 and up row i with
//      lanes 32..63 (a row of 2048 values is 32 block pairs), reduces both and
//      writes act = gelu_tanh(g)*u.  x is staged once per workgroup.
//   3. down: wave s of a workgroup streams the rows of slot s for the
//      workgroup's tile of outputs; partial results meet in LDS and are merged
//      IN SLOT ORDER in f32, as the reference's axpy chain does.
#include "moe_grouped.hpp"
#include "q4_0_mfma.hpp"

namespace {

constexpr int kFlagBadExpertId = 1;
constexpr int kFlagNonFiniteScore = 2;
constexpr uint32_t kScoresMfmaMinTokens = 16;   // from here the router scores run on the f64 matrix cores

// ---------------------------------------------------------------------------
// router
// ---------------------------------------------------------------------------

// DPP lane exchange of a 64-bit value; lanes the control word does not write
// keep their own value.
template <int CTRL, int ROW_MASK = 0xF>
__device__ __forceinline__ double dpp_move_f64(double v) {
    int lo = __double2loint(v), hi = __double2hiint(v);
    lo = __builtin_amdgcn_update_dpp(lo, lo, CTRL, ROW_MASK, 0xF, false);
    hi = __builtin_amdgcn_update_dpp(hi, hi, CTRL, ROW_MASK, 0xF, false);
    return __hiloint2double(hi, lo);
}

__device__ __forceinline__ double lane63_f64(double v) {
    int lo = __builtin_amdgcn_readlane(__double2loint(v), 63);
    int hi = __builtin_amdgcn_readlane(__double2hiint(v), 63);
    return __hiloint2double(hi, lo);
}

// Sum / maximum over the 64 lanes, returned in every lane (wave-uniform).
__device__ __forceinline__ double wave_sum_f64(double v) {
    v += dpp_move_f64<0xB1>(v);
    v += dpp_move_f64<0x4E>(v);
    v += dpp_move_f64<0x141>(v);
    v += dpp_move_f64<0x140>(v);
    {   // row_bcast steps: lanes outside the mask must add nothing
        int lo = __builtin_amdgcn_update_dpp(0, __double2loint(v), 0x142, 0xA, 0xF, false);
        int hi = __builtin_amdgcn_update_dpp(0, __double2hiint(v), 0x142, 0xA, 0xF, false);
        v += __hiloint2double(hi, lo);
        lo = __builtin_amdgcn_update_dpp(0, __double2loint(v), 0x143, 0xC, 0xF, false);
        hi = __builtin_amdgcn_update_dpp(0, __double2hiint(v), 0x143, 0xC, 0xF, false);
        v += __hiloint2double(hi, lo);
    }
    return lane63_f64(v);
}

__device__ __forceinline__ float wave_max_f32(float v) {
#define LEV_MAXSTEP(CTRL, MASK)                                                                   \
    v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(                           \
                     __builtin_bit_cast(int, v), __builtin_bit_cast(int, v), CTRL, MASK, 0xF, false)))
    LEV_MAXSTEP(0xB1, 0xF);
    LEV_MAXSTEP(0x4E, 0xF);
    LEV_MAXSTEP(0x141, 0xF);
    LEV_MAXSTEP(0x140, 0xF);
    LEV_MAXSTEP(0x142, 0xA);
    LEV_MAXSTEP(0x143, 0xC);
#undef LEV_MAXSTEP
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

// Orders one wave's LDS writes before its later LDS reads (the hardware runs
// a wave's LDS accesses in order; this only restrains the compiler).
__device__ __forceinline__ void wave_lds_fence() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// LDS the selection needs: a table of probabilities with 64*J entries (J as the
// selection is instantiated, not the expert count: the layout below is laid
// out for the whole table), as many rank counters, then 64 selected
// probabilities and ids.
__host__ __device__ constexpr size_t router_lds_bytes(uint32_t j) {
    return (size_t)(64u * j) * 12u + 64u * 8u + 64u * 4u;
}
// ... plus the eight waves' partial rank counts of the register-based selection
__host__ __device__ constexpr size_t router_lds_bytes_fast(uint32_t j) {
    return router_lds_bytes(j) + (size_t)8u * (64u * j) * 4u;
}

struct router_sel {
    const double *sel_p;     // LDS: probabilities of the selected experts, selection order
    const uint32_t *sel_id;  // LDS: their indices
    bool ok;                 // false: a score was not finite, nothing selected
    uint32_t e_slot = 0xFFFFFFFFu;   // register-based selection: the expert of the slot asked for;
                                     // sel_p / sel_id are then only filled when need_p was set
};

// softmax (f64) + top-k (ties -> lower index) for one token
// (Gemma4.swift:3798-3810), run by a whole workgroup (every thread calls it;
// blockDim a multiple of 64 and of the padded expert count when that is below
// blockDim).  srow: the token's `experts` scores, written by an earlier kernel.
//
// Repeated extraction of the maximum with ties to the lower index is the same
// as ordering by the strict total order "p larger, or p equal and index
// lower"; an element's rank under that order is the number of elements that
// come before it.  The workgroup counts ranks in parallel: the threads split
// into blockDim/padded parts, each part compares every element against its
// share of the table.
//
// J: each lane of a wave keeps experts j*64+lane, j < J, in registers, and
// every wave computes the whole softmax for itself (same values, same order,
// same result), so the only exchanges are the table, the ranks and the winners.
// need_p = false (uniform over the workgroup): the caller only wants the ids;
// sel_p is then not meaningful.
// The token's scores as every wave holds them: lane l keeps experts j*64 + l.
template <int J>
__device__ __forceinline__ void router_load_scores(const float *__restrict__ srow, uint32_t experts,
                                                   float (&sc)[J]) {
    const uint32_t lane = threadIdx.x & 63u;
#pragma unroll
    for (int j = 0; j < J; ++j) {
        const uint32_t i = lane + 64u * j;
        sc[j] = srow[i < experts ? i : experts - 1u];
    }
}

template <int J>
__device__ router_sel router_select_regs(const float (&sc)[J], void *lds, uint32_t experts,
                                         uint32_t top_k, bool need_p, bool fast, uint32_t slot = 0);

template <int J>
__device__ router_sel router_select_block(const float *__restrict__ srow, void *lds,
                                          uint32_t experts, uint32_t top_k, bool need_p = true) {
    float sc[J];
    router_load_scores<J>(srow, experts, sc);
    return router_select_regs<J>(sc, lds, experts, top_k, need_p, false);
}

// fast (workgroup-uniform, J <= 8): every wave extracts the minima of the integer
// keys from its own registers, round by round, with no exchange at all (see
// below).  Only when the integer keys order the probabilities (the common case);
// the result is the same.
template <int J>
__device__ router_sel router_select_regs(const float (&sc)[J], void *lds, uint32_t experts,
                                         uint32_t top_k, bool need_p, bool fast, uint32_t slot) {
    constexpr uint32_t padded = 64u * J;
    uint64_t *table = static_cast<uint64_t *>(lds);   // probabilities (f64) or order keys
    double *sel_p = reinterpret_cast<double *>(table + padded);
    uint32_t *rank = reinterpret_cast<uint32_t *>(sel_p + 64);
    uint32_t *sel_id = rank + padded;
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    router_sel out{sel_p, sel_id, true, 0xFFFFFFFFu};

    float mx = -INFINITY;
    bool finite = true;
#pragma unroll
    for (int j = 0; j < J; ++j) {
        finite = finite && isfinite(sc[j]);
        mx = fmaxf(mx, sc[j]);
    }
    mx = wave_max_f32(mx);
    if (__any(!finite)) {   // uniform over the workgroup
        out.ok = false;
        return out;
    }
    // The probabilities are exp(d)/sum with d = score - max <= 0 (f32).  While
    // every d is 0 or lies in [-690, -1e-6], two different d are at least 1e-13
    // apart relative to exp's value and every quotient is a normal number, so the
    // probabilities order exactly as the d do and equal d give equal
    // probabilities: the order "p larger, ties to the lower index" is then the
    // ascending order of the integer (|d| bits, index).  Outside that range
    // (exp saturating at 1 or running into denormals) the probabilities
    // themselves are compared.
    uint64_t key[J];
    bool plain = true;
#pragma unroll
    for (int j = 0; j < J; ++j) {
        const uint32_t i = lane + 64u * j;
        const bool valid = i < experts;
        const float d = sc[j] - mx;
        plain = plain && (!valid || d == 0.f || (d <= -1e-6f && d >= -690.f));
        key[j] = valid ? ((uint64_t)(__float_as_uint(d) & 0x7FFFFFFFu) << 32) | i : ~0ull;
    }
    const bool by_key = !__any(!plain);   // every wave holds the same scores: uniform
    const bool with_p = need_p || !by_key;
    double p[J];
    if (with_p) {
        double sum = 0.0;
#pragma unroll
        for (int j = 0; j < J; ++j) {
            const bool valid = lane + 64u * j < experts;
            p[j] = valid ? exp((double)(sc[j] - mx)) : 0.0;   // subtraction in f32, exp in f64
            sum += p[j];
        }
        sum = wave_sum_f64(sum);
#pragma unroll
        for (int j = 0; j < J; ++j) p[j] = lane + 64u * j < experts ? p[j] / sum : 0.0;
    }
    if constexpr (J <= 8) {
        if (fast && by_key) {
            // Repeated extraction of the minimum key, as the reference extracts the
            // maximum probability: every wave holds all keys (two per lane for 128
            // experts) and needs no one else.  A round is a wave-wide minimum of the
            // |d| bits (DPP), a ballot for the lowest index that holds it, and its
            // removal: about twenty instructions.  The workgroup of `slot` stops after
            // slot + 1 rounds; only the publishing workgroup runs all top_k and lists
            // the winners with their probabilities.
            uint32_t dk[J];
#pragma unroll
            for (int j = 0; j < J; ++j) dk[j] = lane + 64u * j < experts ? (uint32_t)(key[j] >> 32) : 0xFFFFFFFFu;
            const uint32_t rounds = need_p ? top_k : slot + 1u;
            uint32_t found = 0xFFFFFFFFu;
            for (uint32_t rnd = 0; rnd < rounds; ++rnd) {
                uint32_t m = dk[0];
#pragma unroll
                for (int j = 1; j < J; ++j) m = dk[j] < m ? dk[j] : m;
#define LEV_MOE_MINSTEP(CTRL, ROWS)                                                                \
                {                                                                                  \
                    const uint32_t o = (uint32_t)__builtin_amdgcn_update_dpp((int)m, (int)m, CTRL, ROWS, 0xF, false); \
                    m = o < m ? o : m;                                                             \
                }
                LEV_MOE_MINSTEP(0xB1, 0xF)    // quad_perm [1,0,3,2]
                LEV_MOE_MINSTEP(0x4E, 0xF)    // quad_perm [2,3,0,1]
                LEV_MOE_MINSTEP(0x141, 0xF)   // row_half_mirror
                LEV_MOE_MINSTEP(0x140, 0xF)   // row_mirror
                LEV_MOE_MINSTEP(0x142, 0xA)   // row_bcast:15 into rows 1 and 3
                LEV_MOE_MINSTEP(0x143, 0xC)   // row_bcast:31 into rows 2 and 3: lane 63 holds the minimum
#undef LEV_MOE_MINSTEP
                const uint32_t best = (uint32_t)__builtin_amdgcn_readlane((int)m, 63);
                uint32_t wl = 0, wj = 0;
                bool seen = false;
#pragma unroll
                for (int j = 0; j < J; ++j) {   // ascending j, lowest lane: the lowest index among equals
                    const unsigned long long hit = __ballot(dk[j] == best);
                    if (!seen && hit != 0ull) {
                        wl = (uint32_t)__builtin_ctzll(hit);
                        wj = (uint32_t)j;
                        seen = true;
                    }
                }
                found = wl + 64u * wj;
#pragma unroll
                for (int j = 0; j < J; ++j) {
                    const bool mine = lane == wl && wj == (uint32_t)j;
                    if (need_p && wave == 0 && mine) {
                        sel_id[rnd] = found;
                        sel_p[rnd] = p[j];
                    }
                    dk[j] = mine ? 0xFFFFFFFFu : dk[j];
                }
            }
            out.e_slot = found;   // need_p: the last winner; the publisher reads sel_id instead
            if (need_p) {
                out.e_slot = 0xFFFFFFFFu;
                lev_barrier_lds();
            }
            return out;
        }
    }
    if (wave == 0) {
#pragma unroll
        for (int j = 0; j < J; ++j) {
            // padding entries (probability 0, or the largest key) sit at indices
            // above every real one: they rank last
            table[lane + 64u * j] = by_key ? key[j] : (uint64_t)__double_as_longlong(p[j]);
            rank[lane + 64u * j] = 0u;
        }
    }
    lev_barrier_lds();
    auto count_before = [&](uint32_t i, uint32_t j0, uint32_t j1) {
        uint32_t before = 0;
        if (by_key) {
            const uint64_t ki = table[i];
#pragma unroll 8
            for (uint32_t j = j0; j < j1; ++j) before += table[j] < ki ? 1u : 0u;
        } else {
            const double pi = __longlong_as_double((long long)table[i]);
#pragma unroll 8
            for (uint32_t j = j0; j < j1; ++j) {
                // same address across the wave: a broadcast read
                const double pj = __longlong_as_double((long long)table[j]);
                before += (pj > pi || (pj == pi && j < i)) ? 1u : 0u;
            }
        }
        return before;
    };
    if (blockDim.x > padded) {
        const uint32_t parts = blockDim.x / padded, share = padded / parts;
        const uint32_t i = tid % padded, part = tid / padded;
        atomicAdd(&rank[i], count_before(i, part * share, (part + 1u) * share));
    } else {
        for (uint32_t i = tid; i < padded; i += blockDim.x) rank[i] = count_before(i, 0u, padded);
    }
    lev_barrier_lds();
    if (wave == 0) {
#pragma unroll
        for (int j = 0; j < J; ++j) {
            const uint32_t i = lane + 64u * j;
            const uint32_t r = rank[i];
            if (i < experts && r < top_k) {
                sel_id[r] = i;
                sel_p[r] = with_p ? p[j] : 0.0;
            }
        }
    }
    lev_barrier_lds();
    return out;
}

// The same selection run by ONE wave with no exchange at all, for kernels in which a single
// wave ranks the scores while the others of the workgroup do something else: the wave holds all
// scores (lane l keeps experts j*64 + l) and extracts minima of the integer keys round by round
// (see router_select_regs).  all == false: returns the expert of `slot` after slot + 1 rounds.
// all == true: lists the top_k winners and their probabilities in sel_id / sel_p (LDS, the layout
// of router_select_regs) and returns the expert of `slot`.
// Returns kRouteNotFinite when a score is not finite, kRouteNeedsBlock when the integer keys do
// not order the probabilities (exp saturating or running into denormals): the caller then runs
// the workgroup-wide selection.
constexpr uint32_t kRouteNotFinite = 0xFFFFFFFFu, kRouteNeedsBlock = 0xFFFFFFFEu;

template <int J>
__device__ uint32_t router_select_wave(const float (&sc)[J], void *lds, uint32_t experts, uint32_t top_k,
                                       uint32_t slot, bool all) {
    constexpr uint32_t padded = 64u * J;
    uint64_t *table = static_cast<uint64_t *>(lds);
    double *sel_p = reinterpret_cast<double *>(table + padded);
    uint32_t *rank = reinterpret_cast<uint32_t *>(sel_p + 64);
    uint32_t *sel_id = rank + padded;
    const uint32_t lane = threadIdx.x & 63u;
    float mx = -INFINITY;
    bool finite = true;
#pragma unroll
    for (int j = 0; j < J; ++j) {
        finite = finite && isfinite(sc[j]);
        mx = fmaxf(mx, sc[j]);
    }
    mx = wave_max_f32(mx);
    if (__any(!finite)) return kRouteNotFinite;
    uint32_t dk[J];
    bool plain = true;
#pragma unroll
    for (int j = 0; j < J; ++j) {
        const bool valid = lane + 64u * j < experts;
        const float d = sc[j] - mx;
        plain = plain && (!valid || d == 0.f || (d <= -1e-6f && d >= -690.f));
        dk[j] = valid ? __float_as_uint(d) & 0x7FFFFFFFu : 0xFFFFFFFFu;
    }
    if (__any(!plain)) return kRouteNeedsBlock;
    double p[J];
    if (all) {
        double sum = 0.0;
#pragma unroll
        for (int j = 0; j < J; ++j) {
            const bool valid = lane + 64u * j < experts;
            p[j] = valid ? exp((double)(sc[j] - mx)) : 0.0;   // subtraction in f32, exp in f64
            sum += p[j];
        }
        sum = wave_sum_f64(sum);
#pragma unroll
        for (int j = 0; j < J; ++j) p[j] = lane + 64u * j < experts ? p[j] / sum : 0.0;
    }
    const uint32_t rounds = all ? top_k : slot + 1u;
    uint32_t mine = 0xFFFFFFFFu;
    for (uint32_t rnd = 0; rnd < rounds; ++rnd) {
        uint32_t m = dk[0];
#pragma unroll
        for (int j = 1; j < J; ++j) m = dk[j] < m ? dk[j] : m;
#define LEV_MOE_MINSTEP(CTRL, ROWS)                                                                \
        {                                                                                          \
            const uint32_t o = (uint32_t)__builtin_amdgcn_update_dpp((int)m, (int)m, CTRL, ROWS, 0xF, false); \
            m = o < m ? o : m;                                                                     \
        }
        LEV_MOE_MINSTEP(0xB1, 0xF)
        LEV_MOE_MINSTEP(0x4E, 0xF)
        LEV_MOE_MINSTEP(0x141, 0xF)
        LEV_MOE_MINSTEP(0x140, 0xF)
        LEV_MOE_MINSTEP(0x142, 0xA)
        LEV_MOE_MINSTEP(0x143, 0xC)
#undef LEV_MOE_MINSTEP
        const uint32_t best = (uint32_t)__builtin_amdgcn_readlane((int)m, 63);
        uint32_t wl = 0, wj = 0;
        bool seen = false;
#pragma unroll
        for (int j = 0; j < J; ++j) {   // ascending j, lowest lane: the lowest index among equals
            const unsigned long long hit = __ballot(dk[j] == best);
            if (!seen && hit != 0ull) {
                wl = (uint32_t)__builtin_ctzll(hit);
                wj = (uint32_t)j;
                seen = true;
            }
        }
        const uint32_t found = wl + 64u * wj;
        if (rnd == slot) mine = found;
#pragma unroll
        for (int j = 0; j < J; ++j) {
            const bool here = lane == wl && wj == (uint32_t)j;
            if (all && here) {
                sel_id[rnd] = found;
                sel_p[rnd] = p[j];
            }
            dk[j] = here ? 0xFFFFFFFFu : dk[j];
        }
    }
    return mine;
}

// Renormalised weight of selection slot k (Gemma4.swift:3808-3810): the sum
// runs over the slots in order, in f64.
__device__ __forceinline__ float router_weight(const router_sel &r, const float *expert_scale,
                                               uint32_t top_k, uint32_t k) {
    double prob_sum = 0.0;
    for (uint32_t m = 0; m < top_k; ++m) prob_sum += r.sel_p[m];
    float wgt = (float)(r.sel_p[k] / prob_sum);
    if (expert_scale) wgt *= expert_scale[r.sel_id[k]];
    return wgt;
}

// Router scores, f64 accumulation rounded to f32 once.  Workgroup (e, g) owns
// router row e.
//   split = 1 (up to four tokens, gridDim.y = 1): the waves share the row, a
//     part of the columns each, for every token, and meet in LDS.
//   split = 0: wave w of group g scores the four tokens 4*(4g+w).. against the
//     row, which it reads once for the four.
constexpr uint32_t kScoreTokensPerWave = 4;

__global__ void __launch_bounds__(256)
moe_scores_kernel(const float *__restrict__ wr, const float *__restrict__ x,
                  float *__restrict__ scores, uint32_t hidden, uint32_t experts, uint32_t tokens,
                  int split) {
    __shared__ double partial[4][4];
    const uint32_t e = blockIdx.x, lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t waves = blockDim.x >> 6;
    const float *row = wr + (uint64_t)e * hidden;
    const bool vec = (hidden & 3u) == 0u &&
                     ((reinterpret_cast<uintptr_t>(wr) | reinterpret_cast<uintptr_t>(x)) & 15u) == 0u;
    if (split) {
        for (uint32_t t = 0; t < tokens; ++t) {
            const float *xv = x + (uint64_t)t * hidden;
            double acc;
            if (vec) {
                const lev_f32x4 *r4 = reinterpret_cast<const lev_f32x4 *>(row);
                const lev_f32x4 *x4 = reinterpret_cast<const lev_f32x4 *>(xv);
                double a0 = 0.0, a1 = 0.0;
                for (uint32_t i = threadIdx.x; i < hidden / 4u; i += blockDim.x) {
                    lev_f32x4 a = r4[i], b = x4[i];
                    a0 = fma((double)a.x, (double)b.x, a0);
                    a1 = fma((double)a.y, (double)b.y, a1);
                    a0 = fma((double)a.z, (double)b.z, a0);
                    a1 = fma((double)a.w, (double)b.w, a1);
                }
                acc = a0 + a1;
            } else {
                acc = 0.0;
                for (uint32_t i = threadIdx.x; i < hidden; i += blockDim.x)
                    acc = fma((double)row[i], (double)xv[i], acc);
            }
            acc = wave_sum_f64(acc);
            if (lane == 0) partial[t][wave] = acc;
        }
        lev_barrier_lds();
        if (threadIdx.x < tokens) {
            double acc = partial[threadIdx.x][0];
            for (uint32_t w = 1; w < waves; ++w) acc += partial[threadIdx.x][w];
            scores[(uint64_t)threadIdx.x * experts + e] = (float)acc;
        }
        return;
    }
    constexpr uint32_t K = kScoreTokensPerWave;
    const uint32_t t0 = (blockIdx.y * waves + wave) * K;
    if (t0 >= tokens) return;
    const float *xv[K];
#pragma unroll
    for (uint32_t k = 0; k < K; ++k)   // tokens past the end repeat the last one and are not stored
        xv[k] = x + (uint64_t)(t0 + k < tokens ? t0 + k : tokens - 1u) * hidden;
    double acc[K] = {};
    if (vec) {
        const lev_f32x4 *r4 = reinterpret_cast<const lev_f32x4 *>(row);
#pragma unroll 4
        for (uint32_t i = lane; i < hidden / 4u; i += 64u) {
            const lev_f32x4 a = r4[i];
#pragma unroll
            for (uint32_t k = 0; k < K; ++k) {
                const lev_f32x4 b = reinterpret_cast<const lev_f32x4 *>(xv[k])[i];
                double lo = fma((double)a.x, (double)b.x, (double)a.y * (double)b.y);
                double hi = fma((double)a.z, (double)b.z, (double)a.w * (double)b.w);
                acc[k] += lo + hi;
            }
        }
    } else {
        for (uint32_t i = lane; i < hidden; i += 64u) {
            const float a = row[i];
#pragma unroll
            for (uint32_t k = 0; k < K; ++k) acc[k] = fma((double)a, (double)xv[k][i], acc[k]);
        }
    }
#pragma unroll
    for (uint32_t k = 0; k < K; ++k) {
        const double total = wave_sum_f64(acc[k]);
        if (lane == 0 && t0 + k < tokens) scores[(uint64_t)(t0 + k) * experts + e] = (float)total;
    }
}

// Many tokens: scores as a small f64 matrix product on the matrix cores
// (v_mfma_f64_16x16x4_f64: exact products of f32 inputs, f64 sums, rounded to
// f32 once by the selection kernel).  A 16-token x 16-expert tile is shared by
// kScoreSplit workgroups of four waves; the sixteen waves split the hidden
// dimension (the loop is latency-bound: a short share per wave keeps all of its
// loads in flight at once, and four workgroups a tile put 128 CUs instead of 32
// to work at 64 tokens x 128 experts).  A workgroup adds its waves' partial
// tiles in wave order and leaves the f64 sum in partials[split][token][expert];
// moe_topk_kernel adds the kScoreSplit of them in order.  The router
// and the activations are each read (tokens/16) resp. (experts/16) times instead
// of once per (expert, 16 tokens).
// Lane (i, kq) = (l % 16, l / 16) loads four consecutive floats of token row i
// and of router row i; MFMA m of a step takes element m of both, i.e. the 16
// k's of a step are spread as k = 4*kq + m: the same permutation on both
// operands.  hidden % 256 == 0, rows 16-byte aligned.
typedef double moe_f64x4 __attribute__((ext_vector_type(4)));

constexpr uint32_t kScoreSplit = 4;

__global__ void __launch_bounds__(256)
moe_scores_mfma_kernel(const float *__restrict__ wr, const float *__restrict__ x, double *__restrict__ partials,
                       uint32_t hidden, uint32_t experts, uint32_t tokens) {
    __shared__ double part[16 / kScoreSplit][256];
    const uint32_t lane = threadIdx.x & 63u, lw = threadIdx.x >> 6;
    const uint32_t wave = blockIdx.z * (16u / kScoreSplit) + lw;   // which sixteenth of the hidden dimension
    const uint32_t i = lane & 15u, kq = lane >> 4;
    const uint32_t e0 = blockIdx.x * 16u, t0 = blockIdx.y * 16u;
    const uint32_t tok = t0 + i < tokens ? t0 + i : tokens - 1u;       // rows past the end repeat the last one
    const uint32_t exp = e0 + i < experts ? e0 + i : experts - 1u;
    const uint32_t span = hidden >> 4;                                  // this wave's share of the hidden dimension
    const lev_f32x4 *xa = reinterpret_cast<const lev_f32x4 *>(x + (uint64_t)tok * hidden + wave * span) + kq;
    const lev_f32x4 *wb = reinterpret_cast<const lev_f32x4 *>(wr + (uint64_t)exp * hidden + wave * span) + kq;
    moe_f64x4 acc = {0.0, 0.0, 0.0, 0.0};
    const uint32_t steps = span >> 4;
    // four steps' operands are requested together (steps past the end repeat the last one with a zero
    // activation: they add nothing)
    for (uint32_t s0 = 0; s0 < steps; s0 += 4u) {
        lev_f32x4 a[4], b[4];
#pragma unroll
        for (uint32_t j = 0; j < 4u; ++j) {
            const uint32_t s = s0 + j < steps ? s0 + j : steps - 1u;
            a[j] = xa[4u * s];
            b[j] = wb[4u * s];
        }
#pragma unroll
        for (uint32_t j = 0; j < 4u; ++j) {
            const bool live = s0 + j < steps;
            const lev_f32x4 aj = live ? a[j] : lev_f32x4{0.f, 0.f, 0.f, 0.f};
            const lev_f32x4 bj = live ? b[j] : lev_f32x4{0.f, 0.f, 0.f, 0.f};
            acc = __builtin_amdgcn_mfma_f64_16x16x4f64((double)aj.x, (double)bj.x, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f64_16x16x4f64((double)aj.y, (double)bj.y, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f64_16x16x4f64((double)aj.z, (double)bj.z, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f64_16x16x4f64((double)aj.w, (double)bj.w, acc, 0, 0, 0);
        }
    }
    // D of the f64 16x16x4 product: register r of lane (i, kq) is row (token) 4*r + kq of column (expert) i
#pragma unroll
    for (int r = 0; r < 4; ++r) part[lw][(4u * (uint32_t)r + kq) * 16u + i] = acc[r];
    lev_barrier_lds();
    const uint32_t tt = (threadIdx.x >> 4) & 15u, ee = threadIdx.x & 15u;
    if (t0 + tt < tokens && e0 + ee < experts) {
        double total = part[0][threadIdx.x];
#pragma unroll
        for (uint32_t w = 1; w < 16u / kScoreSplit; ++w) total += part[w][threadIdx.x];
        partials[((uint64_t)blockIdx.z * tokens + t0 + tt) * experts + e0 + ee] = total;
    }
}

// grid (tokens), 256 threads: selection for one token, written to global memory.
// partials (optional): the scores arrive as kScoreSplit f64 partial sums per (token,
// expert) from moe_scores_mfma_kernel; they are added in order, rounded to f32 once
// and also stored in `scores`.
template <int J>
__global__ void __launch_bounds__(256)
moe_topk_kernel(float *__restrict__ scores, const double *__restrict__ partials,
                const float *__restrict__ expert_scale, int32_t *__restrict__ ids,
                float *__restrict__ weights, int *__restrict__ flag, uint32_t experts, uint32_t top_k,
                uint32_t tokens) {
    extern __shared__ double s_router[];
    const uint32_t t = blockIdx.x;
    router_sel r;
    if (partials) {
        const uint32_t lane = threadIdx.x & 63u;
        float sc[J];
#pragma unroll
        for (int j = 0; j < J; ++j) {
            const uint32_t i = lane + 64u * j, ic = i < experts ? i : experts - 1u;
            double total = partials[(uint64_t)t * experts + ic];
#pragma unroll
            for (uint32_t k = 1; k < kScoreSplit; ++k) total += partials[((uint64_t)k * tokens + t) * experts + ic];
            sc[j] = (float)total;
            if (threadIdx.x < 64u && i < experts) scores[(uint64_t)t * experts + i] = sc[j];
        }
        r = router_select_regs<J>(sc, s_router, experts, top_k, true, false);
    } else {
        r = router_select_block<J>(scores + (uint64_t)t * experts, s_router, experts, top_k);
    }
    if (!r.ok && threadIdx.x == 0) atomicOr(flag, kFlagNonFiniteScore);
    if (threadIdx.x < top_k) {
        ids[(uint64_t)t * top_k + threadIdx.x] = r.ok ? (int32_t)r.sel_id[threadIdx.x] : (int32_t)threadIdx.x;
        weights[(uint64_t)t * top_k + threadIdx.x] =
            r.ok ? router_weight(r, expert_scale, top_k, threadIdx.x) : 0.f;
    }
}

// Up to four tokens: scores AND selection in one launch.  Workgroup (g, t) scores
// experts 8g..8g+7 of token t, one router row per wave (f64 sums, rounded to f32
// once); the last workgroup of a token to finish (an arrival counter per token)
// reads all of the token's scores and runs the selection, so that the gate/up
// kernel starts from finished ids instead of every one of its workgroups ranking
// the scores for itself.  Sixteen workgroups per token keep the counter short (a
// counter over one workgroup per expert would serialise 128 arrivals).  The
// counter is zero again when the kernel ends.  A forge candidate, not the built-in
// choice: see lev_moe_layer_candidates.
template <int J>
__global__ void __launch_bounds__(512)
moe_scores_select_kernel(const float *__restrict__ wr, const float *__restrict__ x, float *scores,
                         const float *__restrict__ expert_scale, int32_t *__restrict__ ids,
                         float *__restrict__ weights, int *__restrict__ flag, uint32_t *tickets,
                         uint32_t hidden, uint32_t experts, uint32_t top_k) {
    extern __shared__ double s_router[];
    __shared__ uint32_t s_ticket;
    __shared__ float s_score[8];
    const uint32_t t = blockIdx.y, tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t e = blockIdx.x * 8u + wave;
    if (e < experts) {   // wave-uniform
        const float *row = wr + (uint64_t)e * hidden;
        const float *xv = x + (uint64_t)t * hidden;
        double acc;
        if ((hidden & 3u) == 0u &&
            ((reinterpret_cast<uintptr_t>(wr) | reinterpret_cast<uintptr_t>(x)) & 15u) == 0u) {
            const lev_f32x4 *r4 = reinterpret_cast<const lev_f32x4 *>(row);
            const lev_f32x4 *x4 = reinterpret_cast<const lev_f32x4 *>(xv);
            double a0 = 0.0, a1 = 0.0;
#pragma unroll 8
            for (uint32_t i = lane; i < hidden / 4u; i += 64u) {
                const lev_f32x4 a = r4[i], b = x4[i];
                a0 = fma((double)a.x, (double)b.x, a0);
                a1 = fma((double)a.y, (double)b.y, a1);
                a0 = fma((double)a.z, (double)b.z, a0);
                a1 = fma((double)a.w, (double)b.w, a1);
            }
            acc = a0 + a1;
        } else {
            acc = 0.0;
            for (uint32_t i = lane; i < hidden; i += 64u) acc = fma((double)row[i], (double)xv[i], acc);
        }
        acc = wave_sum_f64(acc);
        if (lane == 0) s_score[wave] = (float)acc;
    }
    lev_barrier_lds();
    // One wave stores the workgroup's eight scores with device-scope stores, which go
    // through to memory, waits for them and takes the workgroup's arrival number (a
    // fence in their place writes back every dirty line of the XCD's L2).
    if (wave == 0) {
        const uint32_t eo = blockIdx.x * 8u + lane;
        if (lane < 8u && eo < experts)
            __hip_atomic_store(&scores[(uint64_t)t * experts + eo], s_score[lane], __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
        lev_publish_wait();
        if (lane == 0)
            s_ticket = __hip_atomic_fetch_add(&tickets[t], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (s_ticket != gridDim.x - 1u) return;
    if (tid == 0) __hip_atomic_store(&tickets[t], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // the other workgroups' scores are read with device-scope loads below
    float sc[J];
#pragma unroll
    for (int j = 0; j < J; ++j) {
        const uint32_t i = lane + 64u * j;
        sc[j] = __hip_atomic_load(&scores[(uint64_t)t * experts + (i < experts ? i : experts - 1u)],
                                  __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    const router_sel r = router_select_regs<J>(sc, s_router, experts, top_k, true, true, 0u);
    if (!r.ok && tid == 0) atomicOr(flag, kFlagNonFiniteScore);
    if (tid < top_k) {
        ids[(uint64_t)t * top_k + tid] = r.ok ? (int32_t)r.sel_id[tid] : (int32_t)tid;
        weights[(uint64_t)t * top_k + tid] = r.ok ? router_weight(r, expert_scale, top_k, tid) : 0.f;
    }
}

// ---------------------------------------------------------------------------
// expert ids: bounds + distinctness (MoEModelBinding.offsets requires both)
// ---------------------------------------------------------------------------

// The token's selection is usable for `slot` when its id is an expert and no
// other slot names the same one.  Run by a whole wave (top_k <= 64): lane k
// reads ids[k], so the check costs one memory round trip however many slots
// there are.
__device__ __forceinline__ int32_t expert_ids_request(const int32_t *ids, uint32_t top_k) {
    const uint32_t lane = threadIdx.x & 63u;
    return ids[lane < top_k ? lane : top_k - 1u];
}

__device__ __forceinline__ bool expert_ids_verdict(int32_t mine, uint32_t top_k, uint32_t slot,
                                                   uint32_t experts, uint32_t *expert) {
    const uint32_t lane = threadIdx.x & 63u;
    const int32_t me = __builtin_amdgcn_readlane(mine, slot);
    const unsigned long long same = __ballot(lane < top_k && mine == me);
    *expert = (uint32_t)me;
    return me >= 0 && (uint32_t)me < experts && __popcll(same) == 1;
}

__device__ __forceinline__ bool expert_ids_ok(const int32_t *ids, uint32_t top_k, uint32_t slot,
                                              uint32_t experts, uint32_t *expert) {
    const uint32_t lane = threadIdx.x & 63u;
    const int32_t mine = ids[lane < top_k ? lane : top_k - 1u];
    const int32_t me = __builtin_amdgcn_readlane(mine, slot);
    const unsigned long long same = __ballot(lane < top_k && mine == me);
    *expert = (uint32_t)me;
    return me >= 0 && (uint32_t)me < experts && __popcll(same) == 1;
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

constexpr int kGuThreads = 512;
constexpr int kGuWaves = kGuThreads / LEV_WAVE;

// Loads rows i0 + r (r < R) of the lane's half (gate or up): P pairs each.
// Branch-free: rows and pairs past the end are clamped to valid ones.
template <int P, int R>
__device__ __forceinline__ void gu_load_rows(const uint8_t *__restrict__ wbase, uint64_t row_bytes,
                                             uint32_t i0, uint32_t inter, uint32_t pairs, uint32_t lp,
                                             uint32_t D[P][R][9]) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const uint32_t i = i0 + r;
        const uint8_t *rp = wbase + (uint64_t)(i < inter ? i : inter - 1u) * row_bytes;
#pragma unroll
        for (int p = 0; p < P; ++p) {
            const uint32_t pr = lp + 32u * p;
            lev_q4_load_pair(rp + (uint64_t)(pr < pairs ? pr : pairs - 1u) * 36u, D[p][r]);
        }
    }
}

template <int P, int R>
__device__ __forceinline__ void gu_finish_rows(const uint32_t D[P][R][9], const lev_q4_pair_x X[P],
                                               float *__restrict__ arow, uint32_t i0, uint32_t i_end,
                                               uint32_t lane) {
    float mine = 0.f;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        float acc = 0.f;
#pragma unroll
        for (int p = 0; p < P; ++p) acc += lev_q4_pair_dot(D[p][r], X[p]);
        acc = lev_group_sum<32>(acc);
        float g = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, acc), 31));
        float u = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, acc), 63));
        float v = lev_gelu_up_value(g, u);
        mine = lane == (uint32_t)r ? v : mine;
    }
    if (lane < (uint32_t)R && i0 + lane < i_end) arow[i0 + lane] = mine;   // R consecutive floats
}

// grid (chunks_per_slot, top_k, tokens), 8 waves.  Lanes 0..31 of a wave walk
// gate row i and lanes 32..63 up row i; a wave has R such rows in flight and a
// lane covers P pairs of each (rows of up to 64*32*P values).
// ROUTE > 0 (the selection's register count, experts <= 64*ROUTE): the expert
// ids come from this token's router scores, selected here by
// the workgroup itself (every workgroup of a token repeats the selection, which
// costs less than a kernel boundary); the first workgroup of a token publishes
// ids and weights.  Otherwise the ids are read from `ids`.
template <int P, int R, int NS, int ROUTE>
__global__ void __launch_bounds__(kGuThreads)
moe_gate_up_kernel(moe_args a, const float *__restrict__ x, const int32_t *ids,
                   const float *__restrict__ scores, const float *__restrict__ expert_scale,
                   int32_t *ids_out, float *weights_out, float *__restrict__ act,
                   int *__restrict__ flag, uint32_t rows_per_block) {
    extern __shared__ lev_f32x4 xs[];
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t slot = blockIdx.y, t = blockIdx.z;
    const uint32_t pairs = a.hidden / 64u;
    const uint32_t half = lane >> 5, lp = lane & 31u;
    float *bsum = reinterpret_cast<float *>(xs + 16u * (pairs + 1u));
    const float *xt = x + (uint64_t)t * a.hidden;

    // Request order = return order on a CU (its memory pipeline hands data back in
    // the order it was asked for): the scores, which the expert id and with it
    // every weight address hang on, go out first, the activations second.
    float sc[ROUTE > 0 ? ROUTE : 1];
    if constexpr (ROUTE > 0) router_load_scores<ROUTE>(scores + (uint64_t)t * a.experts, a.experts, sc);
    lev_f32x4 xv[NS];
    lev_q4_stage_x_load<NS>(xt, pairs, tid, kGuThreads, xv);

    uint32_t e;
    router_sel r{nullptr, nullptr, true, 0xFFFFFFFFu};
    if constexpr (ROUTE > 0) {
        // 8-byte aligned as it stands: xs is 16-byte aligned and 2*pairs floats
        // follow 16*(pairs+1) vectors.  (Rounding the address up through an
        // integer would hide from the compiler that this is LDS.)
        void *rl = bsum + 2u * pairs;
        // only the workgroup that publishes the selection needs the probabilities
        r = router_select_regs<ROUTE>(sc, rl, a.experts, a.top_k, blockIdx.x == 0 && slot == 0, true, slot);
        e = !r.ok ? slot : r.e_slot != 0xFFFFFFFFu ? r.e_slot : r.sel_id[slot];
    } else {
        const int32_t *tids = ids + (uint64_t)t * a.top_k;
        if (!expert_ids_ok(tids, a.top_k, slot, a.experts, &e)) {
            if (tid == 0) atomicOr(flag, kFlagBadExpertId);
            return;
        }
    }
    const uint64_t row_bytes = (uint64_t)pairs * 36u;
    const uint8_t *wbase = a.base + (half ? a.up_off + e * a.up_stride : a.gate_off + e * a.gate_stride);
    const uint32_t i_begin = blockIdx.x * rows_per_block;
    const uint32_t i_end = min(i_begin + rows_per_block, a.inter);
    constexpr uint32_t kStep = kGuWaves * R;

    uint32_t Da[P][R][9], Db[P][R][9];
    uint32_t i0 = i_begin + wave * R;
    // The activations were requested before anything else and have landed by
    // now: they go to LDS before the weight requests leave, so that the wait for
    // them cannot end up behind the weights.
    lev_q4_stage_x_store_sums<NS>(xt, xs, bsum, pairs, tid, kGuThreads, xv);
    gu_load_rows<P, R>(wbase, row_bytes, i0, a.inter, pairs, lp, Da);
    lev_barrier_lds();
    if constexpr (ROUTE > 0) {
        // the first workgroup of a token publishes the selection while its
        // weights are on their way
        if (blockIdx.x == 0 && slot == 0) {
            if (!r.ok && tid == 0) atomicOr(flag, kFlagNonFiniteScore);
            if (tid < a.top_k) {
                ids_out[(uint64_t)t * a.top_k + tid] = r.ok ? (int32_t)r.sel_id[tid] : (int32_t)tid;
                weights_out[(uint64_t)t * a.top_k + tid] =
                    r.ok ? router_weight(r, expert_scale, a.top_k, tid) : 0.f;
            }
        }
    }

    lev_q4_pair_x X[P];
#pragma unroll
    for (int p = 0; p < P; ++p) {
        const uint32_t pr = lp + 32u * p;
        const bool p_ok = pr < pairs;
        lev_q4_fetch_x_sums(xs, bsum, pairs, p_ok ? pr : pairs - 1u, X[p]);
#pragma unroll
        for (int q = 0; q < 16; ++q) X[p].xr[q] = p_ok ? X[p].xr[q] : lev_f32x4{0.f, 0.f, 0.f, 0.f};
        X[p].sum_a = p_ok ? X[p].sum_a : 0.f;   // padding lanes contribute nothing
        X[p].sum_b = p_ok ? X[p].sum_b : 0.f;
    }
    float *arow = act + ((uint64_t)t * a.top_k + slot) * a.inter;
    if (rows_per_block <= kStep) {   // one step per wave: nothing to prefetch
        gu_finish_rows<P, R>(Da, X, arow, i0, i_end, lane);
        return;
    }
    // unconditional prefetch (clamped past the end): a branch around the loads
    // would make the compiler wait for them before the current rows are used
    while (true) {
        uint32_t next = i0 + kStep;
        gu_load_rows<P, R>(wbase, row_bytes, next, a.inter, pairs, lp, Db);
        gu_finish_rows<P, R>(Da, X, arow, i0, i_end, lane);
        if (next >= i_end) break;
        i0 = next;
        next = i0 + kStep;
        gu_load_rows<P, R>(wbase, row_bytes, next, a.inter, pairs, lp, Da);
        gu_finish_rows<P, R>(Db, X, arow, i0, i_end, lane);
        if (next >= i_end) break;
        i0 = next;
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
// top_k*tile partial sums, then the top_k routing weights.
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
    // the routing weights are requested now and parked in LDS for the merge at
    // the end (top_k <= 64: one lane each)
    float *w_slot = partial + a.top_k * tile;
    const float w_mine = weights[(uint64_t)t * a.top_k + (lane < a.top_k ? lane : a.top_k - 1u)];

    bool bad = false;
    for (uint32_t slot = wave; slot < a.top_k; slot += kDnWaves) {
        // request order = return order: the ids (the weight addresses hang on them)
        // first, then this slot's activations, so that both are on their way while
        // the id is checked and neither waits behind the weights
        const int32_t ids_mine = expert_ids_request(tids, a.top_k);
        const float *av = act + ((uint64_t)t * a.top_k + slot) * a.inter;
        lev_f32x4 av4[kLevStageSlots];
        lev_q4_stage_x_load<kLevStageSlots>(av, pairs, lane, 64u, av4);
        uint32_t e;
        if (!expert_ids_verdict(ids_mine, a.top_k, slot, a.experts, &e)) {
            bad = true;
            for (uint32_t r = lane; r < tile; r += 64u) partial[slot * tile + r] = 0.f;
            continue;
        }
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
        lev_q4_stage_x_store<kLevStageSlots>(av, xs, pairs, lane, 64u, av4);
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
    if (wave == 0 && lane < a.top_k) w_slot[lane] = w_mine;
    lev_barrier_lds();
    // ordered merge: y = sum over slots, in slot order, of w_slot * dn[slot]
    for (uint32_t r = tid; r < tile; r += kDnThreads) {
        uint32_t row = row_begin + r;
        if (row >= a.hidden) continue;
        float accum = 0.f;
        for (uint32_t slot = 0; slot < a.top_k; ++slot)
            accum = fmaf(w_slot[slot], partial[slot * tile + r], accum);
        y[(uint64_t)t * a.hidden + row] = accum;
    }
}

// ---------------------------------------------------------------------------
// gate/up and down on the integer matrix cores (q4_0_mfma.hpp), up to four tokens.
// A task is 16 rows x 256 activations; a wave stages the activations of its own tasks in LDS of
// its own (no workgroup barrier in front of the products) and keeps the operands in registers.
// ---------------------------------------------------------------------------

constexpr int kMmWaves = 8;
constexpr int kMmThreads = kMmWaves * LEV_WAVE;
constexpr uint32_t kGumPartBytes = 2u * 2u * kMmWaves * 16u * 4u;   // [round parity][gate, up][wave][row] f32

__host__ __device__ constexpr size_t mm_areas_bytes(uint32_t tpw) {
    return (size_t)kMmWaves * (tpw * kQ4mTaskArea + kQ4mZeroBytes);
}

// grid (chunks, top_k, tokens), 8 waves.  Wave w multiplies the column tasks w*TPW.. of gate row
// group i AND of up row group i (the same operands); the eight partial sums of a row meet in LDS
// and wave 0 writes act = gelu_tanh(g) * u.  A workgroup takes rows_per_block rows in groups of 16
// with the next group's weights in flight.
// ROUTE > 0 (experts <= 64*ROUTE): the expert comes from this token's router scores, ranked by
// wave 0 alone while the other waves' activation requests are on their way (every workgroup of a
// token repeats the selection, which costs less than a kernel boundary; one wave ranking costs an
// eighth of the vector instructions of eight); the first workgroup of a token publishes ids and
// weights.  Otherwise the ids are read from `ids`.
// LDS: part | expert word | task areas | router area (ROUTE > 0)
template <int TPW, int ROUTE>
__global__ void __launch_bounds__(kMmThreads)
moe_gate_up_mfma(moe_args a, const float *__restrict__ x, const int32_t *ids, const float *__restrict__ scores,
                 const float *__restrict__ expert_scale, int32_t *ids_out, float *weights_out,
                 float *__restrict__ act, int *__restrict__ flag, uint32_t rows_per_block) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const uint32_t slot = blockIdx.y, t = blockIdx.z;
    const uint32_t ntask = a.hidden >> 8;
    const uint32_t t_first = wave * TPW;
    const float *xt = x + (uint64_t)t * a.hidden;

    // request order = return order: the scores (the expert, and with it every weight address,
    // hangs on them) first, the activations behind them
    float sc[ROUTE > 0 ? ROUTE : 1];
    if constexpr (ROUTE > 0) {
        if (wave == 0u) router_load_scores<ROUTE>(scores + (uint64_t)t * a.experts, a.experts, sc);
    }
    lev_f32x4 v[TPW];
#pragma unroll
    for (int k = 0; k < TPW; ++k) {
        const uint32_t T = t_first + k < ntask ? t_first + k : ntask - 1u;
        v[k] = reinterpret_cast<const lev_f32x4 *>(xt)[64u * T + lane];
    }

    uint32_t *s_e = reinterpret_cast<uint32_t *>(smem + kGumPartBytes);
    uint8_t *area = smem + kGumPartBytes + 16u + (size_t)wave * (TPW * kQ4mTaskArea + kQ4mZeroBytes);
    uint8_t *zero = area + TPW * kQ4mTaskArea;
    void *rl = smem + kGumPartBytes + 16u + mm_areas_bytes(TPW);
    uint32_t e;
    bool ok = true;
    const bool publisher = ROUTE > 0 && blockIdx.x == 0 && slot == 0;
    if constexpr (ROUTE > 0) {
        // (all eight waves ranking a share of the keys each was measured as well: the layer takes 0.5 us
        // longer, the 16 waves of a CU then queue for its four vector pipelines)
        if (wave == 0u) {
            const uint32_t got = router_select_wave<ROUTE>(sc, rl, a.experts, a.top_k, slot, publisher);
            if (lane == 0u) s_e[0] = got;
        }
        lev_barrier_lds();
        e = s_e[0];
        if (e == kRouteNeedsBlock) {   // workgroup-uniform and rare: the workgroup ranks the probabilities together
            const router_sel r = router_select_block<ROUTE>(scores + (uint64_t)t * a.experts, rl, a.experts,
                                                            a.top_k, publisher);
            e = r.ok ? r.sel_id[slot] : kRouteNotFinite;
        }
        ok = e != kRouteNotFinite;
        if (!ok) e = slot;
    } else {
        const int32_t *tids = ids + (uint64_t)t * a.top_k;
        if (!expert_ids_ok(tids, a.top_k, slot, a.experts, &e)) {
            if (tid == 0) atomicOr(flag, kFlagBadExpertId);
            return;
        }
    }
    e = (uint32_t)__builtin_amdgcn_readfirstlane((int)e);
    const uint64_t row_bytes = (uint64_t)(a.hidden >> 6) * 36u;
    const uint8_t *gbase = a.base + a.gate_off + e * a.gate_stride;
    const uint8_t *ubase = a.base + a.up_off + e * a.up_stride;
    const uint32_t i_begin = blockIdx.x * rows_per_block;
    const uint32_t i_end = min(i_begin + rows_per_block, a.inter);
    const uint32_t lrow = lane >> 2;                              // fetch order: lane = 4 * row + pair
    auto issue = [&](uint32_t i0, uint32_t (&Dg)[TPW][9], uint32_t (&Du)[TPW][9]) {
        uint32_t row = i0 + lrow;
        row = row < i_end ? row : i_end - 1u;
        const uint64_t off = (uint64_t)row * row_bytes;
#pragma unroll
        for (int k = 0; k < TPW; ++k) {
            const uint32_t T = t_first + k < ntask ? t_first + k : ntask - 1u;
            q4m_load_task(gbase + off, 4u * T, Dg[k]);
            q4m_load_task(ubase + off, 4u * T, Du[k]);
        }
    };
    uint32_t Ga[TPW][9], Ua[TPW][9];
    uint32_t i0 = i_begin;
    issue(i0, Ga, Ua);

    // ---- while the weights are on their way ----
    if constexpr (ROUTE > 0) {
        if (publisher) {
            constexpr uint32_t padded = 64u * ROUTE;
            uint64_t *table = static_cast<uint64_t *>(rl);
            double *sel_p = reinterpret_cast<double *>(table + padded);
            uint32_t *sel_id = reinterpret_cast<uint32_t *>(sel_p + 64) + padded;
            const router_sel r{sel_p, sel_id, ok, 0xFFFFFFFFu};
            if (!ok && tid == 0) atomicOr(flag, kFlagNonFiniteScore);
            if (tid < a.top_k) {
                ids_out[(uint64_t)t * a.top_k + tid] = ok ? (int32_t)sel_id[tid] : (int32_t)tid;
                weights_out[(uint64_t)t * a.top_k + tid] = ok ? router_weight(r, expert_scale, a.top_k, tid) : 0.f;
            }
        }
    }
    const uint32_t r16 = lane & 15u, q = lane >> 4;
    uint32_t pw = (wave * 16u + lane) * 4u;                       // byte offsets into `part`: gate, then up at + 512
    uint32_t pr = (q * 16u + r16) * 4u;                           // wave 0: lane (r, q) adds waves q and q + 4
    float *arow = act + ((uint64_t)t * a.top_k + slot) * a.inter;
    lev_pin(pw);
    lev_pin(pr);
    if (lane < kQ4mZeroBytes / 4u) reinterpret_cast<uint32_t *>(zero)[lane] = 0u;
    q4m_operand op[TPW];
#pragma unroll
    for (int k = 0; k < TPW; ++k) q4m_stage_task(v[k], area + k * kQ4mTaskArea, zero, t_first + k < ntask, op[k]);
    __builtin_amdgcn_sched_barrier(0);

    auto finish = [&](uint32_t i_here, const uint32_t (&Dg)[TPW][9], const uint32_t (&Du)[TPW][9]) {
        float vg = 0.f, vu = 0.f;
#pragma unroll
        for (int k = 0; k < TPW; ++k) {
            uint32_t W[9];
            q4m_turn_task(Dg[k], W);
            vg += q4m_task_dot(W, op[k]);
            q4m_turn_task(Du[k], W);
            vu += q4m_task_dot(W, op[k]);
        }
        vg = q4m_row_sum(vg);
        vu = q4m_row_sum(vu);
        if (lane < 16u) {
            *reinterpret_cast<float *>(smem + pw) = vg;
            *reinterpret_cast<float *>(smem + pw + kMmWaves * 16u * 4u) = vu;
        }
        lev_barrier_lds();
        if (wave == 0u) {
            const float *pp = reinterpret_cast<const float *>(smem + pr);
            const float g0 = pp[0], g1 = pp[64], u0 = pp[128], u1 = pp[192];
            const float g = q4m_row_sum(g0 + g1), u = q4m_row_sum(u0 + u1);
            if (q == 0u && i_here + r16 < i_end) arow[i_here + r16] = lev_gelu_up_value(g, u);
        }
        pw ^= kGumPartBytes / 2u;                                 // the other half of `part` next round
        pr ^= kGumPartBytes / 2u;
    };
    if (rows_per_block <= 16u) {   // one group per workgroup: nothing to prefetch
        finish(i0, Ga, Ua);
        return;
    }
    // unconditional (clamped) prefetch: a branch around the loads would make the compiler wait
    // for them before the current group is multiplied
    uint32_t Gb[TPW][9], Ub[TPW][9];
    while (true) {
        uint32_t next = i0 + 16u;
        issue(next < i_end ? next : i0, Gb, Ub);
        finish(i0, Ga, Ua);
        if (next >= i_end) break;
        i0 = next;
        next = i0 + 16u;
        issue(next < i_end ? next : i0, Ga, Ua);
        finish(i0, Gb, Ub);
        if (next >= i_end) break;
        i0 = next;
    }
}

// grid (row tiles of `tile` <= 16 rows, tokens), 8 waves.  Wave s takes slots s, s + 8, ...: the
// whole reduction (TPW tasks, inter <= 256*TPW) of the tile's rows against the slot's activations,
// which it stages for itself; the per-slot results meet in LDS and are merged IN SLOT ORDER in
// f32, as the reference's axpy chain does.
// LDS: partial [top_k][16] f32 | w_slot [64] f32 | task areas
template <int TPW>
__global__ void __launch_bounds__(kMmThreads)
moe_down_mfma(moe_args a, const float *__restrict__ act, const int32_t *__restrict__ ids,
              const float *__restrict__ weights, float *__restrict__ y, int *__restrict__ flag, uint32_t tile) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const uint32_t t = blockIdx.y;
    const uint32_t ntask = a.inter >> 8;
    const uint32_t row_begin = blockIdx.x * tile;
    const uint32_t row_end = min(row_begin + tile, a.hidden);
    float *partial = reinterpret_cast<float *>(smem);                       // [top_k][16]
    float *w_slot = partial + a.top_k * 16u;
    uint8_t *area = smem + (size_t)a.top_k * 64u + 256u + (size_t)wave * (TPW * kQ4mTaskArea + kQ4mZeroBytes);
    uint8_t *zero = area + TPW * kQ4mTaskArea;
    const int32_t *tids = ids + (uint64_t)t * a.top_k;
    const uint64_t row_bytes = (uint64_t)(a.inter >> 6) * 36u;
    // the routing weights are requested now and parked in LDS for the merge at the end
    const float w_mine = weights[(uint64_t)t * a.top_k + (lane < a.top_k ? lane : a.top_k - 1u)];
    if (lane < kQ4mZeroBytes / 4u) reinterpret_cast<uint32_t *>(zero)[lane] = 0u;
    uint32_t lr = row_begin + (lane >> 2);                                   // fetch order: lane = 4 * row + pair
    lr = lr < row_end ? lr : row_end - 1u;

    bool bad = false;
    for (uint32_t slot = wave; slot < a.top_k; slot += kMmWaves) {
        // request order = return order: the ids (the weight addresses hang on them) first, then
        // this slot's activations
        const int32_t ids_mine = expert_ids_request(tids, a.top_k);
        const float *av = act + ((uint64_t)t * a.top_k + slot) * a.inter;
        lev_f32x4 v[TPW];
#pragma unroll
        for (int k = 0; k < TPW; ++k) {
            const uint32_t T = (uint32_t)k < ntask ? (uint32_t)k : ntask - 1u;
            v[k] = reinterpret_cast<const lev_f32x4 *>(av)[64u * T + lane];
        }
        uint32_t e;
        if (!expert_ids_verdict(ids_mine, a.top_k, slot, a.experts, &e)) {
            bad = true;
            if (lane < 16u) partial[slot * 16u + lane] = 0.f;
            continue;
        }
        e = (uint32_t)__builtin_amdgcn_readfirstlane((int)e);
        const uint8_t *rowp = a.base + a.down_off + e * a.down_stride + (uint64_t)lr * row_bytes;
        uint32_t D[TPW][9];
#pragma unroll
        for (int k = 0; k < TPW; ++k) {
            const uint32_t T = (uint32_t)k < ntask ? (uint32_t)k : ntask - 1u;
            q4m_load_task(rowp, 4u * T, D[k]);
        }
        // the slot's activations become operands while its weights are on their way
        q4m_operand op[TPW];
#pragma unroll
        for (int k = 0; k < TPW; ++k) q4m_stage_task(v[k], area + k * kQ4mTaskArea, zero, (uint32_t)k < ntask, op[k]);
        __builtin_amdgcn_sched_barrier(0);
        float val = 0.f;
#pragma unroll
        for (int k = 0; k < TPW; ++k) {
            uint32_t W[9];
            q4m_turn_task(D[k], W);
            val += q4m_task_dot(W, op[k]);
        }
        val = q4m_row_sum(val);
        if (lane < 16u) partial[slot * 16u + lane] = val;
    }
    if (bad && lane == 0) atomicOr(flag, kFlagBadExpertId);
    if (wave == 0u && lane < a.top_k) w_slot[lane] = w_mine;
    lev_barrier_lds();
    // ordered merge: y = sum over slots, in slot order, of w_slot * dn[slot]
    if (tid < 16u && row_begin + tid < row_end) {
        float accum = 0.f;
        // eight slots' reads in flight together, the multiply-adds in slot order behind them
        for (uint32_t s0 = 0; s0 < a.top_k; s0 += 8u) {
            float pv[8], wv[8];
#pragma unroll
            for (uint32_t u = 0; u < 8u; ++u) {
                const uint32_t slot = s0 + u < a.top_k ? s0 + u : a.top_k - 1u;
                pv[u] = partial[slot * 16u + tid];
                wv[u] = w_slot[slot];
            }
#pragma unroll
            for (uint32_t u = 0; u < 8u; ++u)
                if (s0 + u < a.top_k) accum = fmaf(wv[u], pv[u], accum);
        }
        y[(uint64_t)t * a.hidden + row_begin + tid] = accum;
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
    uint32_t e;
    if (!expert_ids_ok(tids, a.top_k, slot, a.experts, &e)) {
        if (threadIdx.x == 0) atomicOr(flag, kFlagBadExpertId);
        return;
    }
    if (i >= a.inter) return;
    const uint32_t blocks = a.hidden / 32u;
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
        uint32_t e;
        if (!expert_ids_ok(tids, a.top_k, slot, a.experts, &e)) {
            if (lane == 0) atomicOr(flag, kFlagBadExpertId);
            continue;
        }
        float d = q4_0_row_dot_generic(
            a.base + a.down_off + e * a.down_stride + (uint64_t)row * blocks * 18u,
            act + ((uint64_t)t * a.top_k + slot) * a.inter, blocks, lane);
        accum = fmaf(weights[(uint64_t)t * a.top_k + slot], d, accum);
    }
    if (lane == 0) y[(uint64_t)t * a.hidden + row] = accum;
}

constexpr uint32_t kRouteInKernelMax = 256;   // experts the gate/up kernel selects by itself

// Where the expert ids of the gate/up kernel come from.
struct gu_route {
    const int32_t *ids;          // given ids, or NULL: select from scores
    const float *scores, *expert_scale;
    int32_t *ids_out;
    float *weights_out;
};

template <int P, int R, int NS>
hipError_t launch_gate_up(lev_ctx *ctx, const moe_args &a, const float *x, const gu_route &rt,
                          float *act, uint32_t tokens, uint32_t per_cu) {
    // rows per workgroup: about per_cu (two, unless a schedule says otherwise)
    // workgroups per CU at one token, more rows per workgroup (less re-staging of x) at many
    constexpr uint32_t step = kGuWaves * R;
    uint64_t slots = (uint64_t)a.top_k * tokens;
    uint32_t want_blocks_per_slot = (uint32_t)(((uint64_t)ctx->num_cus * per_cu + slots - 1) / slots);
    if (want_blocks_per_slot < 1) want_blocks_per_slot = 1;
    // (not rounded to whole steps: with 12 rows per workgroup half of its waves take
    // a second row, which beats 16 rows on three quarters of the workgroups)
    uint32_t rows_per_block = (a.inter + want_blocks_per_slot - 1) / want_blocks_per_slot;
    (void)step;
    uint32_t chunks = (a.inter + rows_per_block - 1) / rows_per_block;
    const uint32_t pairs = a.hidden / 64u;
    size_t lds = (size_t)16 * (pairs + 1u) * sizeof(lev_f32x4) + (size_t)2 * pairs * sizeof(float);
    dim3 grid(chunks, a.top_k, tokens);
    if (rt.ids) {
        hipLaunchKernelGGL((moe_gate_up_kernel<P, R, NS, 0>), grid, dim3(kGuThreads), lds, ctx->stream,
                           a, x, rt.ids, nullptr, nullptr, nullptr, nullptr, act, ctx->d_flag,
                           rows_per_block);
    } else {
        lds += 8 + router_lds_bytes_fast(a.experts <= 128u ? 2u : 4u);
        if (a.experts <= 128u)
            hipLaunchKernelGGL((moe_gate_up_kernel<P, R, NS, 2>), grid, dim3(kGuThreads), lds, ctx->stream,
                               a, x, nullptr, rt.scores, rt.expert_scale, rt.ids_out, rt.weights_out,
                               act, ctx->d_flag, rows_per_block);
        else   // callers keep experts <= kRouteInKernelMax
            hipLaunchKernelGGL((moe_gate_up_kernel<P, R, NS, 4>), grid, dim3(kGuThreads), lds, ctx->stream,
                               a, x, nullptr, rt.scores, rt.expert_scale, rt.ids_out, rt.weights_out,
                               act, ctx->d_flag, rows_per_block);
    }
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
    if (steps < 1) steps = 1;
    if (steps > 64) steps = 64;
    tile = steps * G;
    uint32_t tiles = (a.hidden + tile - 1) / tile;
    size_t lds = (size_t)kDnWaves * 16 * (a.inter / 64u + 1u) * sizeof(lev_f32x4) +
                 (size_t)a.top_k * (tile + 1u) * sizeof(float);
    if (lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&moe_down_kernel<L>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL((moe_down_kernel<L>), dim3(tiles, tokens), dim3(kDnThreads), lds, ctx->stream,
                       a, act, ids, weights, y, ctx->d_flag, steps);
    return hipGetLastError();
}

// Shapes the matrix-core expert kernels take: rows of whole 256-value tasks, at most two tasks a
// wave for gate/up (the hidden dimension is split over the eight waves), at most four for down
// (a wave reduces over the whole intermediate dimension).
bool gate_up_mfma_ok(const moe_args &a) { return a.hidden % 256u == 0u && a.hidden <= 4096u; }
bool down_mfma_ok(const moe_args &a) { return a.inter % 256u == 0u && a.inter <= 1024u; }

hipError_t launch_gate_up_mfma(lev_ctx *ctx, const moe_args &a, const float *x, const gu_route &rt,
                               float *act, uint32_t tokens, uint32_t per_cu) {
    const uint64_t slots = (uint64_t)a.top_k * tokens;
    uint32_t want = (uint32_t)(((uint64_t)ctx->num_cus * per_cu + slots - 1) / slots);
    if (want < 1) want = 1;
    const uint32_t rows_per_block = (a.inter + want - 1) / want;
    const uint32_t chunks = (a.inter + rows_per_block - 1) / rows_per_block;
    const uint32_t tpw = a.hidden > 2048u ? 2u : 1u;
    const uint32_t route = rt.ids ? 0u : a.experts <= 128u ? 2u : 4u;      // callers keep experts <= kRouteInKernelMax
    const size_t lds = kGumPartBytes + 16u + mm_areas_bytes(tpw) + (route ? router_lds_bytes(route) + 8u : 0u);
    const dim3 grid(chunks, a.top_k, tokens);
#define LEV_GUM(TPW, ROUTE)                                                                          \
    hipLaunchKernelGGL((moe_gate_up_mfma<TPW, ROUTE>), grid, dim3(kMmThreads), lds, ctx->stream, a, x, rt.ids,   \
                       rt.scores, rt.expert_scale, rt.ids_out, rt.weights_out, act, ctx->d_flag, rows_per_block)
    if (tpw == 1u) {
        if (route == 0u) LEV_GUM(1, 0);
        else if (route == 2u) LEV_GUM(1, 2);
        else LEV_GUM(1, 4);
    } else {
        if (route == 0u) LEV_GUM(2, 0);
        else if (route == 2u) LEV_GUM(2, 2);
        else LEV_GUM(2, 4);
    }
#undef LEV_GUM
    return hipGetLastError();
}

hipError_t launch_down_mfma(lev_ctx *ctx, const moe_args &a, const float *act, const int32_t *ids,
                            const float *weights, float *y, uint32_t tokens) {
    // one workgroup per CU at one token; a tile is at most the 16 rows of a task
    uint32_t want_tiles = (uint32_t)(((uint64_t)ctx->num_cus + tokens - 1) / tokens);
    if (want_tiles < 1) want_tiles = 1;
    uint32_t tile = (a.hidden + want_tiles - 1) / want_tiles;
    tile = tile < 4u ? 4u : tile > 16u ? 16u : tile;
    const uint32_t tiles = (a.hidden + tile - 1) / tile;
    const uint32_t tpw = (a.inter + 255u) / 256u;
    const size_t lds = (size_t)a.top_k * 64u + 256u + mm_areas_bytes(tpw);
    const dim3 grid(tiles, tokens);
#define LEV_DNM(TPW)                                                                                 \
    hipLaunchKernelGGL((moe_down_mfma<TPW>), grid, dim3(kMmThreads), lds, ctx->stream, a, act, ids, weights, y, \
                       ctx->d_flag, tile)
    if (tpw == 1u) LEV_DNM(1);
    else if (tpw == 2u) LEV_DNM(2);
    else if (tpw == 3u) LEV_DNM(3);
    else LEV_DNM(4);
#undef LEV_DNM
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

bool experts_fast(const moe_args &a, const float *x) {
    auto al4 = [&](uint64_t v) { return ((reinterpret_cast<uintptr_t>(a.base) + v) & 3u) == 0; };
    return a.hidden % 64u == 0 && a.inter % 64u == 0 && a.hidden <= 4096u && a.inter <= 4096u &&
           al4(a.gate_off) && al4(a.up_off) && al4(a.down_off) && a.gate_stride % 4u == 0 &&
           a.up_stride % 4u == 0 && a.down_stride % 4u == 0 &&
           (reinterpret_cast<uintptr_t>(x) & 15u) == 0;
}

// rt.ids == NULL (selection inside the gate/up kernel) is only valid on the
// fast path: callers test experts_fast() first.
hipError_t run_experts(lev_ctx *ctx, const moe_args &a, const float *x, const gu_route &rt,
                       const int32_t *ids, const float *weights, float *y, float *act,
                       uint32_t tokens, bool fast, uint32_t gu_per_cu = 2u, bool matrix_cores = true) {
    hipError_t e;
    if (!fast) {
        hipLaunchKernelGGL(moe_gate_up_generic, dim3((a.inter + 3) / 4, a.top_k, tokens), dim3(256), 0,
                           ctx->stream, a, x, ids, act, ctx->d_flag);
        if ((e = hipGetLastError()) != hipSuccess) return e;
        hipLaunchKernelGGL(moe_down_generic, dim3((a.hidden + 3) / 4, tokens), dim3(256), 0,
                           ctx->stream, a, act, ids, weights, y, ctx->d_flag);
        return hipGetLastError();
    }
    // One row pair per wave and step: what a wave does after its last byte has
    // landed is issued at one instruction per eight cycles whatever else runs
    // on the SIMD, so many short waves finish sooner than few long ones.
    static const bool env_mfma = [] {
        const char *v = getenv("LEV_MOE_MFMA");   // LEV_MOE_MFMA=0: the vector-ALU expert kernels, for comparison
        return !(v && v[0] == '0');
    }();
    const bool mfma = matrix_cores && env_mfma;
    if (mfma && gate_up_mfma_ok(a)) e = launch_gate_up_mfma(ctx, a, x, rt, act, tokens, gu_per_cu);
    else if (a.hidden <= 2048u) e = launch_gate_up<1, 1, 1>(ctx, a, x, rt, act, tokens, gu_per_cu);
    else e = launch_gate_up<2, 1, 2>(ctx, a, x, rt, act, tokens, gu_per_cu);
    if (e != hipSuccess) return e;
    if (mfma && down_mfma_ok(a)) return launch_down_mfma(ctx, a, act, ids, weights, y, tokens);
    const uint32_t dp = a.inter / 64u;
    if (dp > 32) return launch_down<64>(ctx, a, act, ids, weights, y, tokens);
    if (dp > 16) return launch_down<32>(ctx, a, act, ids, weights, y, tokens);
    if (dp > 8) return launch_down<16>(ctx, a, act, ids, weights, y, tokens);
    if (dp > 4) return launch_down<8>(ctx, a, act, ids, weights, y, tokens);
    return launch_down<4>(ctx, a, act, ids, weights, y, tokens);
}

// scratch layout: [scores f32[tokens*experts] | f64 partial scores [kScoreSplit][tokens*experts] from
// kScoresMfmaMinTokens tokens | act f32[tokens*top_k*inter] | grouped work area]
struct moe_scratch {
    float *scores;
    double *partials;   // nullptr below kScoresMfmaMinTokens tokens
    float *act;
    void *grouped;   // work area of the many-token path (grouped_bytes > 0)
};

size_t score_partial_bytes(uint32_t tokens, uint32_t experts) {
    return tokens >= kScoresMfmaMinTokens ? (((size_t)kScoreSplit * tokens * experts * 8 + 255) & ~(size_t)255) : 0;
}

int get_scratch(lev_ctx *ctx, uint32_t tokens, uint32_t experts, uint32_t top_k, uint32_t inter,
                moe_scratch *s, size_t grouped_bytes = 0) {
    size_t s_bytes = ((size_t)tokens * experts * 4 + 255) & ~(size_t)255;
    size_t p_bytes = score_partial_bytes(tokens, experts);
    size_t a_bytes = ((size_t)tokens * top_k * inter * 4 + 255) & ~(size_t)255;
    char *p = static_cast<char *>(lev_scratch(ctx, s_bytes + p_bytes + a_bytes + grouped_bytes));
    if (!p) return lev_fail(ctx, LEV_ERR_EXCEEDS_WORKING_SET, "moe: scratch allocation failed");
    s->scores = reinterpret_cast<float *>(p);
    s->partials = p_bytes ? reinterpret_cast<double *>(p + s_bytes) : nullptr;
    s->act = reinterpret_cast<float *>(p + s_bytes + p_bytes);
    s->grouped = p + s_bytes + p_bytes + a_bytes;
    return LEV_OK;
}

// Tokens from which pairs are grouped by expert and multiplied on the matrix
// cores; below, every (token, slot) streams its expert by itself.
constexpr uint32_t kGroupedMinTokens = 5;

lev_moe_grouped_args grouped_args(const moe_args &a, uint32_t tokens) {
    return lev_moe_grouped_args{a.base,        a.gate_off,  a.up_off, a.down_off, a.gate_stride,
                                a.up_stride,   a.down_stride, a.hidden, a.inter,   a.experts,
                                a.top_k,       tokens};
}

bool use_grouped(const lev_ctx *ctx, const moe_args &a, const float *x, uint32_t tokens) {
    static const bool enabled = [] {
        const char *e = getenv("LEV_MOE_GROUPED");   // LEV_MOE_GROUPED=0: per-pair kernels, for comparison
        return !(e && e[0] == '0');
    }();
    return enabled && tokens >= kGroupedMinTokens && experts_fast(a, x) &&
           lev_moe_grouped_usable(ctx, grouped_args(a, tokens));
}

// *in_partials: the scores were left as f64 partial sums in `partials` (for run_topk), not in `scores`.
hipError_t run_scores(lev_ctx *ctx, const float *wr, const float *x, float *scores, double *partials,
                      bool *in_partials, uint32_t hidden, uint32_t experts, uint32_t tokens) {
    *in_partials = false;
    if (partials && tokens >= kScoresMfmaMinTokens && hidden % 256u == 0u &&
        ((reinterpret_cast<uintptr_t>(wr) | reinterpret_cast<uintptr_t>(x)) & 15u) == 0u) {
        hipLaunchKernelGGL(moe_scores_mfma_kernel, dim3((experts + 15u) / 16u, (tokens + 15u) / 16u, kScoreSplit),
                           dim3(256), 0, ctx->stream, wr, x, partials, hidden, experts, tokens);
        *in_partials = true;
        return hipGetLastError();
    }
    const int split = tokens <= 4u;
    const uint32_t per_group = 4u * kScoreTokensPerWave;
    const uint32_t groups = split ? 1u : (tokens + per_group - 1u) / per_group;
    hipLaunchKernelGGL(moe_scores_kernel, dim3(experts, groups), dim3(256), 0, ctx->stream, wr, x,
                       scores, hidden, experts, tokens, split);
    return hipGetLastError();
}

// scores and selection in one launch (tokens <= 4, experts <= kRouteInKernelMax)
hipError_t run_scores_select(lev_ctx *ctx, const float *wr, const float *x, float *scores, const float *scale,
                             int32_t *ids, float *weights, uint32_t hidden, uint32_t experts, uint32_t top_k,
                             uint32_t tokens) {
    uint32_t *tickets = reinterpret_cast<uint32_t *>(ctx->d_flag) + lev_ctx::kTicketWord;
    const dim3 grid((experts + 7u) / 8u, tokens);
    if (experts <= 128u)
        hipLaunchKernelGGL((moe_scores_select_kernel<2>), grid, dim3(512), router_lds_bytes_fast(2), ctx->stream, wr,
                           x, scores, scale, ids, weights, ctx->d_flag, tickets, hidden, experts, top_k);
    else
        hipLaunchKernelGGL((moe_scores_select_kernel<4>), grid, dim3(512), router_lds_bytes_fast(4), ctx->stream, wr,
                           x, scores, scale, ids, weights, ctx->d_flag, tickets, hidden, experts, top_k);
    return hipGetLastError();
}

hipError_t run_topk(lev_ctx *ctx, float *scores, const double *partials, const float *scale, int32_t *ids,
                    float *weights, uint32_t experts, uint32_t top_k, uint32_t tokens) {
#define LEV_TOPK(J)                                                                               \
    hipLaunchKernelGGL((moe_topk_kernel<J>), dim3(tokens), dim3(256), router_lds_bytes(J), ctx->stream, \
                       scores, partials, scale, ids, weights, ctx->d_flag, experts, top_k, tokens)
    if (experts <= 128u) LEV_TOPK(2);
    else if (experts <= 256u) LEV_TOPK(4);
    else if (experts <= 1024u) LEV_TOPK(16);
    else {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&moe_topk_kernel<64>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize,
                                           (int)router_lds_bytes(64));
        if (e != hipSuccess) return e;
        LEV_TOPK(64);
    }
#undef LEV_TOPK
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
    float *scores = d_scores;
    moe_scratch s{nullptr, nullptr, nullptr, nullptr};
    if (!scores || tokens >= kScoresMfmaMinTokens) {
        int st = get_scratch(ctx, tokens, experts, top_k, 0, &s);
        if (st != LEV_OK) return st;
        if (!scores) scores = s.scores;
    }
    bool in_partials = false;
    int st = lev_hip_check(ctx,
                           run_scores(ctx, d_router_w, d_x, scores, s.partials, &in_partials, hidden, experts,
                                      tokens),
                           "moe router scores launch");
    if (st != LEV_OK) return st;
    return lev_hip_check(ctx,
                         run_topk(ctx, scores, in_partials ? s.partials : nullptr, d_expert_scale, d_ids,
                                  d_weights, experts, top_k, tokens),
                         "moe router top-k launch");
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
    const bool grouped = use_grouped(ctx, a, d_x, tokens) && (reinterpret_cast<uintptr_t>(d_act) & 15u) == 0u;
    float *act = d_act;
    moe_scratch s{nullptr, nullptr, nullptr};
    if (!act || grouped) {
        st = get_scratch(ctx, tokens, a.experts, top_k, a.inter, &s,
                         grouped ? lev_moe_grouped_scratch_bytes(grouped_args(a, tokens)) : 0);
        if (st != LEV_OK) return st;
        if (!act) act = s.act;
    }
    if (grouped)
        return lev_hip_check(ctx,
                             lev_moe_grouped_launch(ctx, grouped_args(a, tokens), d_x, d_ids, d_weights,
                                                    d_y, act, s.grouped),
                             "moe grouped experts launch");
    const bool fast = experts_fast(a, d_x) && (reinterpret_cast<uintptr_t>(act) & 15u) == 0u;
    gu_route rt{d_ids, nullptr, nullptr, nullptr, nullptr};
    return lev_hip_check(ctx, run_experts(ctx, a, d_x, rt, d_ids, d_weights, d_y, act, tokens, fast),
                         "moe experts launch");
}

namespace {

// Whole MoE block.  `fixed` == nullptr: the scratch comes from the context
// (allocated or grown on demand).  Otherwise the caller supplies `fixed_bytes`
// of device memory and nothing is allocated: shapes that need more, or the
// many-token grouped path (which sizes a work area from the routing), are
// refused.
int moe_layer_impl(lev_ctx *ctx, const lev_moe_experts *pools, const float *d_router_w,
                   const float *d_expert_scale, const float *d_x, float *d_y, int32_t *d_ids,
                   float *d_weights, uint32_t top_k, uint32_t tokens, void *fixed, size_t fixed_bytes) {
    if (!d_router_w || !d_x || !d_y || !d_ids || !d_weights)
        return lev_fail(ctx, LEV_ERR_INVALID_ARGUMENT, "moe_layer: null pointer");
    moe_args a;
    int st = check_pools(ctx, pools, top_k, tokens, &a);
    if (st != LEV_OK) return st;
    if (a.experts > 4096u) return lev_fail(ctx, LEV_ERR_BAD_DIMENSIONS, "moe_layer: %u experts", a.experts);
    const bool grouped = !fixed && use_grouped(ctx, a, d_x, tokens);
    moe_scratch s;
    if (fixed) {
        if (tokens > LEV_NOALLOC_MOE_MAX_TOKENS)
            return lev_fail(ctx, LEV_ERR_EXCEEDS_WORKING_SET,
                            "moe_layer_noalloc: %u tokens, at most %u", tokens, LEV_NOALLOC_MOE_MAX_TOKENS);
        const size_t s_bytes = ((size_t)tokens * a.experts * 4 + 255) & ~(size_t)255;
        const size_t a_bytes = ((size_t)tokens * top_k * a.inter * 4 + 255) & ~(size_t)255;
        if (s_bytes + a_bytes > fixed_bytes)
            return lev_fail(ctx, LEV_ERR_EXCEEDS_WORKING_SET,
                            "moe_layer_noalloc: needs %zu bytes of scratch, the static buffer holds %zu",
                            s_bytes + a_bytes, fixed_bytes);
        s.scores = static_cast<float *>(fixed);
        s.partials = nullptr;   // at most LEV_NOALLOC_MOE_MAX_TOKENS tokens: the f32 score kernel
        s.act = reinterpret_cast<float *>(static_cast<char *>(fixed) + s_bytes);
        s.grouped = nullptr;
    } else {
        st = get_scratch(ctx, tokens, a.experts, top_k, a.inter, &s,
                         grouped ? lev_moe_grouped_scratch_bytes(grouped_args(a, tokens)) : 0);
        if (st != LEV_OK) return st;
    }
    const bool fast = experts_fast(a, d_x);
    gu_route rt{d_ids, nullptr, nullptr, nullptr, nullptr};
    // a schedule installed for this shape (lev_hip_forge_select) overrides the built-in choice
    const lev_schedule *sel = tokens <= 4u ? lev_selected(ctx, LEV_OP_MOE_LAYER_Q4_0, a.hidden, a.inter, tokens)
                                           : nullptr;
    const uint32_t family = sel ? sel->family : 1u;
    const uint32_t gu_per_cu = sel && sel->rows_in_flight ? sel->rows_in_flight : 2u;
    const bool matrix_cores = !(sel && sel->persistent);   // schedule field `persistent` = 1: the vector-ALU expert kernels
    const bool few = fast && tokens <= 4u && a.experts <= kRouteInKernelMax;
    if (few && family == 2u) {
        // few tokens: the router kernel's last workgroup selects the experts
        st = lev_hip_check(ctx,
                           run_scores_select(ctx, d_router_w, d_x, s.scores, d_expert_scale, d_ids, d_weights,
                                             a.hidden, a.experts, top_k, tokens),
                           "moe router launch");
        if (st != LEV_OK) return st;
    } else {
        bool in_partials = false;
        st = lev_hip_check(ctx,
                           run_scores(ctx, d_router_w, d_x, s.scores, s.partials, &in_partials, a.hidden,
                                      a.experts, tokens),
                           "moe router scores launch");
        if (st != LEV_OK) return st;
        if (few && family == 1u) {
            // the gate/up workgroups select the experts themselves
            rt = gu_route{nullptr, s.scores, d_expert_scale, d_ids, d_weights};
        } else {
            st = lev_hip_check(ctx,
                               run_topk(ctx, s.scores, in_partials ? s.partials : nullptr, d_expert_scale, d_ids,
                                        d_weights, a.experts, top_k, tokens),
                               "moe router top-k launch");
            if (st != LEV_OK) return st;
        }
    }
    if (grouped)
        return lev_hip_check(ctx,
                             lev_moe_grouped_launch(ctx, grouped_args(a, tokens), d_x, d_ids, d_weights,
                                                    d_y, s.act, s.grouped),
                             "moe grouped experts launch");
    return lev_hip_check(ctx,
                         run_experts(ctx, a, d_x, rt, d_ids, d_weights, d_y, s.act, tokens, fast, gu_per_cu, matrix_cores),
                         "moe experts launch");
}

}  // namespace

// Candidate schedules of the MoE layer at one to four tokens, the built-in choice
// first (MoELoweringForge.forge, MoELowering.swift:1896-1985, derives and gates the
// lowered layer the same way): who selects the experts (family 1: the gate/up
// workgroups themselves, the built-in choice; 2: the last workgroup of the router
// kernel to finish; 0: a top-k kernel of its own, one launch more) and how many
// gate/up workgroups per CU the rows are cut into.  On MI355X the hand-over inside
// the router kernel (a fence and an arrival counter over 16 workgroups) costs as
// much as the launch it saves: 18.8 us a layer against 15.9 and 18.9.  Every candidate computes each row with the same lanes in the same order:
// their outputs agree bit for bit.  (Shapes the streaming kernels cannot take run
// the generic kernels whatever is selected.)
uint32_t lev_moe_layer_candidates(const lev_ctx *ctx, uint32_t hidden, uint32_t inter, uint32_t tokens,
                                  lev_schedule *out, uint32_t capacity) {
    (void)ctx;
    (void)hidden;
    (void)inter;
    (void)tokens;
    uint32_t n = 0;
    auto add = [&](uint32_t family, uint32_t per_cu) {
        if (n < capacity) out[n] = lev_schedule{LEV_OP_MOE_LAYER_Q4_0, family, per_cu, 0u};
        ++n;
    };
    add(1u, 2u);
    add(1u, 1u);
    add(1u, 4u);
    add(2u, 2u);
    add(0u, 2u);
    // the expert kernels on the vector ALU (f32 FMA chains) instead of the integer matrix cores, the
    // built-in choice wherever rows are whole 256-value tasks: same routing, sums rounded differently
    if (n < capacity) out[n] = lev_schedule{LEV_OP_MOE_LAYER_Q4_0, 1u, 2u, 1u};
    ++n;
    return n;
}

extern "C" int lev_hip_moe_layer_q4_0(lev_ctx *ctx, const lev_moe_experts *pools,
                                      const float *d_router_w, const float *d_expert_scale,
                                      const float *d_x, float *d_y, int32_t *d_ids, float *d_weights,
                                      uint32_t top_k, uint32_t tokens) {
    LEV_REQUIRE_CTX(ctx);
    return moe_layer_impl(ctx, pools, d_router_w, d_expert_scale, d_x, d_y, d_ids, d_weights, top_k,
                          tokens, nullptr, 0);
}

// ---------------------------------------------------------------------------
// The same block for callers that cannot allocate (code under HIP graph
// capture, serving loops, harnesses that forbid hipMalloc): the router scores
// and the expert activations live in a file-scope device array instead of the
// context's grow-on-demand buffer.  Every GPU holds its own copy of the array
// until the process ends; every call on a GPU uses that one copy, so calls
// that overlap on one GPU (two contexts, two streams) race.  Both regions are
// written in full before they are read, so nothing has to start at zero.
// ---------------------------------------------------------------------------

static __device__ __align__(256) unsigned char lev_moe_static_scratch_array[LEV_NOALLOC_MOE_SCRATCH_BYTES];

// Set-up: called by lev_hip_ctx_create with the context's device current.  The
// array's name is only a host-side handle; its device address differs per GPU
// and comes from the runtime.
int lev_moe_static_scratch_init(lev_ctx *ctx) {
    void *p = nullptr;
    hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(lev_moe_static_scratch_array));
    if (e != hipSuccess || !p) {
        ctx->moe_static_scratch = nullptr;
        return lev_hip_check(ctx, e != hipSuccess ? e : hipErrorInvalidSymbol, "hipGetSymbolAddress(static MoE scratch)");
    }
    ctx->moe_static_scratch = p;
    return LEV_OK;
}

extern "C" int lev_hip_moe_layer_q4_0_noalloc(lev_ctx *ctx, const lev_moe_experts *pools,
                                              const float *d_router_w, const float *d_expert_scale,
                                              const float *d_x, float *d_y, int32_t *d_ids,
                                              float *d_weights, uint32_t top_k, uint32_t tokens) {
    LEV_REQUIRE_CTX(ctx);
    if (!ctx->moe_static_scratch)
        return lev_fail(ctx, LEV_ERR_DEVICE_UNAVAILABLE, "moe_layer_noalloc: the static scratch has no device address");
    return moe_layer_impl(ctx, pools, d_router_w, d_expert_scale, d_x, d_y, d_ids, d_weights, top_k,
                          tokens, ctx->moe_static_scratch, LEV_NOALLOC_MOE_SCRATCH_BYTES);
}

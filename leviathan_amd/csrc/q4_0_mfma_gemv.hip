// Q4_0 decode GEMV  y = W x  on the integer matrix cores (gfx950).
//
// Stands in for g4_q4_matvec and its tiled / generated variants
// (Sources/LeviathanCore/Gemma4.swift:3931, 4031; Q4Lowering.swift:541-664) wherever a row is a
// whole number of 256-value tasks; q4_0_gemv.hip keeps the vector-ALU kernels for every other
// shape and as forge candidates.
//
// Workgroup = 16 waves.  A row group is 16 rows; its in_dim / 256 column tasks are split over
// WPR waves, TPW adjacent tasks each (WPR * TPW >= tasks).  Rows narrower than 16 tasks leave
// room for 16 / WPR row groups per round of the workgroup.  A wave stages the activations of its
// own tasks once, keeps the operands in registers and walks the row groups of its slot with the
// next group's weights in flight; the WPR partial sums of a row meet in LDS behind ONE barrier a
// round, and the wave of the slot adds them in a fixed order.
#include "q4_0_mfma.hpp"

namespace {

constexpr int kQ4mWaves = 16;
constexpr int kQ4mThreads = kQ4mWaves * LEV_WAVE;

// LDS: part [2][16 waves][16 rows] f32 (2 KB, so that the round's half is one XOR away) | per
// wave TPW task areas and a zero strip
__host__ __device__ constexpr size_t q4m_gemv_lds(uint32_t tpw) {
    return 2u * kQ4mWaves * 16u * 4u + (size_t)kQ4mWaves * (tpw * kQ4mTaskArea + kQ4mZeroBytes);
}

// wave -> (slot, position in the slot): 4-bit entries of two 64-bit kernel arguments (lev_wave_tables).
// SINGLE: the grid covers every round once: straight-line code, nothing to prefetch.
template <int TPW, bool SINGLE>
__global__ void __launch_bounds__(kQ4mThreads)
q4_0_mfma_gemv(const uint8_t *__restrict__ w, const float *__restrict__ x, float *__restrict__ y,
               uint32_t in_dim, uint32_t rows, uint32_t wpr, uint32_t slots, uint64_t slot_of_wave,
               uint64_t pos_of_wave) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    // wave-uniform by construction: in a scalar register, so that everything derived from it is
    // scalar arithmetic
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const uint32_t slot = (uint32_t)(slot_of_wave >> (4u * wave)) & 15u;   // idle waves: slot >= slots
    const uint32_t tw = (uint32_t)(pos_of_wave >> (4u * wave)) & 15u;
    const uint32_t ntask = in_dim >> 8;
    const uint32_t t_first = tw * TPW;

    // the activations of the wave's tasks first (short, mostly L2 hits) ...
    lev_f32x4 v[TPW];
#pragma unroll
    for (int t = 0; t < TPW; ++t) {
        const uint32_t T = t_first + t < ntask ? t_first + t : ntask - 1u;
        v[t] = reinterpret_cast<const lev_f32x4 *>(x)[64u * T + lane];
    }
    // ... the first row group's weights right behind them
    const bool active = slot < slots;
    const uint64_t row_bytes = (uint64_t)(in_dim >> 6) * 36u;
    const uint32_t ngroups = (rows + 15u) >> 4;
    const uint32_t lrow = lane >> 2;                             // fetch order: lane = 4 * row + pair
    auto issue = [&](uint32_t round_block, uint32_t (&D)[TPW][9]) {
        uint32_t rg = round_block * slots + (active ? slot : 0u);
        rg = rg < ngroups ? rg : ngroups - 1u;
        uint32_t row = rg * 16u + lrow;
        row = row < rows ? row : rows - 1u;
        const uint8_t *rowp = w + (uint64_t)row * row_bytes;
#pragma unroll
        for (int t = 0; t < TPW; ++t) {
            const uint32_t T = t_first + t < ntask ? t_first + t : ntask - 1u;
            q4m_load_task(rowp, 4u * T, D[t]);
        }
    };
    uint32_t Da[TPW][9];
    uint32_t rb = blockIdx.x;
    issue(rb, Da);

    // ---- everything the tail of a round needs, while the loads are on their way ----
    uint8_t *area = smem + 2u * kQ4mWaves * 16u * 4u + (size_t)wave * (TPW * kQ4mTaskArea + kQ4mZeroBytes);
    uint8_t *zero = area + TPW * kQ4mTaskArea;                  // the wave's own: no barrier before the staging
    const uint32_t r = lane & 15u, q = lane >> 4;
    // the wave's partial sums: lanes 0..15 write row `lane`
    // (byte offsets into the workgroup's LDS, not pointers: an address that has been through an
    // integer register is no longer known to be LDS)
    uint32_t pw = (wave * 16u + lane) * 4u;
    // wave s < slots adds the wpr partial sums of slot s: lane (r, q) reads waves q, q + 4, q + 8, q + 12
    // of the slot (those past the slot's waves are masked after the read)
    uint32_t pr = (((wave < slots ? wave : 0u) * wpr + q) * 16u + r) * 4u;
    uint32_t k0 = q < wpr ? ~0u : 0u, k1 = q + 4u < wpr ? ~0u : 0u, k2 = q + 8u < wpr ? ~0u : 0u,
             k3 = q + 12u < wpr ? ~0u : 0u;
    uint32_t orow = (rb * slots + wave) * 16u + r;
    const uint32_t orow_step = gridDim.x * slots * 16u;
    const bool writer = wave < slots && q == 0u;
    uint32_t stores = writer && orow < rows ? 1u : 0u;
    uint64_t yp = reinterpret_cast<uint64_t>(y + orow);        // (the pointer argument is read here, not behind the barrier)
    lev_pin(pw);
    lev_pin(pr);
    lev_pin(k0);
    lev_pin(k1);
    lev_pin(k2);
    lev_pin(k3);
    lev_pin(stores);
    lev_pin(yp);

    if (lane < kQ4mZeroBytes / 4u) reinterpret_cast<uint32_t *>(zero)[lane] = 0u;
    q4m_operand op[TPW];
#pragma unroll
    for (int t = 0; t < TPW; ++t)
        q4m_stage_task(v[t], area + t * kQ4mTaskArea, zero, active && t_first + t < ntask, op[t]);
    // the operands are read back before the wait for the weights, not behind it
    __builtin_amdgcn_sched_barrier(0);

    const uint32_t nrounds = (ngroups + slots - 1u) / slots;     // rounds of `slots` row groups
    auto finish = [&](const uint32_t (&D)[TPW][9]) {
        float val = 0.f;
#pragma unroll
        for (int t = 0; t < TPW; ++t) {
            uint32_t W[9];
            q4m_turn_task(D[t], W);
            val += q4m_task_dot(W, op[t]);
        }
        val = q4m_row_sum(val);
        if (lane < 16u) *reinterpret_cast<float *>(smem + pw) = val;
        lev_barrier_lds();
        if (wave < slots) {
            const float *pp = reinterpret_cast<const float *>(smem + pr);
            const float p0 = pp[0], p1 = pp[64], p2 = pp[128], p3 = pp[192];   // four reads in flight together
            auto keep = [](float p, uint32_t k) { return __uint_as_float(__float_as_uint(p) & k); };
            float s = (keep(p0, k0) + keep(p1, k1)) + (keep(p2, k2) + keep(p3, k3));
            s = q4m_row_sum(s);
            if (stores) *reinterpret_cast<__attribute__((address_space(1))) float *>(yp) = s;   // a global store, not a flat one
        }
        if (!SINGLE) {
            pw ^= kQ4mWaves * 16u * 4u;                          // the other half of `part` next round
            pr ^= kQ4mWaves * 16u * 4u;
            orow += orow_step;
            yp += (uint64_t)orow_step * 4u;
            stores = writer && orow < rows ? 1u : 0u;
        }
    };
    if (SINGLE) {
        finish(Da);
        return;
    }
    // Unconditional (clamped) prefetch: a branch around the loads would make the compiler wait
    // for them before the current group is multiplied.
    uint32_t Db[TPW][9];
    while (true) {
        uint32_t next = rb + gridDim.x;
        issue(next < nrounds ? next : rb, Db);
        finish(Da);
        if (next >= nrounds) break;
        rb = next;
        next = rb + gridDim.x;
        issue(next < nrounds ? next : rb, Da);
        finish(Db);
        if (next >= nrounds) break;
        rb = next;
    }
}

template <int TPW>
hipError_t launch(lev_ctx *ctx, const uint8_t *w, const float *x, float *y, uint32_t in_dim, uint32_t rows,
                  uint32_t wpr, uint32_t slots, int persistent) {
    const uint32_t ngroups = (rows + 15u) / 16u;
    const uint32_t nrounds = (ngroups + slots - 1u) / slots;
    const size_t lds = q4m_gemv_lds(TPW);
    uint64_t slot_of_wave, pos_of_wave;
    lev_wave_tables(wpr, &slot_of_wave, &pos_of_wave);
    // built-in choice (persistent < 0): one workgroup per round while every round has a CU of its own
    const uint32_t cus = (uint32_t)ctx->num_cus;
    const bool single = persistent < 0 ? nrounds <= cus : persistent == 0;
    if (single) {
        if (lds > 48 * 1024) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&q4_0_mfma_gemv<TPW, true>),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return e;
        }
        hipLaunchKernelGGL((q4_0_mfma_gemv<TPW, true>), dim3(nrounds), dim3(kQ4mThreads), lds, ctx->stream, w, x, y,
                           in_dim, rows, wpr, slots, slot_of_wave, pos_of_wave);
        return hipGetLastError();
    }
    if (lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&q4_0_mfma_gemv<TPW, false>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
    }
    const uint32_t blocks = nrounds < cus ? nrounds : cus;
    hipLaunchKernelGGL((q4_0_mfma_gemv<TPW, false>), dim3(blocks), dim3(kQ4mThreads), lds, ctx->stream, w, x, y,
                       in_dim, rows, wpr, slots, slot_of_wave, pos_of_wave);
    return hipGetLastError();
}

}  // namespace

// Shapes the matrix-core GEMV takes: rows of whole 256-value tasks, at most two tasks a wave
// (the operands of more do not fit the 128 registers a wave of a 16-wave workgroup has).
bool lev_q4_0_mfma_gemv_usable(const uint8_t *w, const float *x, uint32_t in_dim) {
    return in_dim % 256u == 0u && in_dim != 0u && in_dim <= kLevQ4MfmaMaxInDim &&
           (reinterpret_cast<uintptr_t>(w) & 3u) == 0u && (reinterpret_cast<uintptr_t>(x) & 15u) == 0u;
}

// persistent: 0 = one workgroup per round of row groups, 1 = resident grid, < 0 = built-in choice.
hipError_t lev_q4_0_mfma_gemv_launch(lev_ctx *ctx, const uint8_t *w, const float *x, float *y, uint32_t in_dim,
                                     uint32_t rows, int persistent) {
    const uint32_t ntask = in_dim >> 8;
    if (ntask <= (uint32_t)kQ4mWaves) {
        // one task per wave; 16 / ntask row groups share a round
        const uint32_t slots = (uint32_t)kQ4mWaves / ntask;
        return launch<1>(ctx, w, x, y, in_dim, rows, ntask, slots, persistent);
    }
    return launch<2>(ctx, w, x, y, in_dim, rows, (ntask + 1u) / 2u, 1u, persistent);
}

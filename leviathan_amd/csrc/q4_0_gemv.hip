// Q4_0 decode GEMV  y = W x  for gfx950.
//
// Stands in for g4_q4_matvec and its tiled / generated variants
// (Sources/LeviathanCore/Gemma4.swift:3931, 4031; Q4Lowering.swift:541-664).
//
// HBM-bound: W is streamed exactly once (18 bytes per 32 weights), x is staged
// once per workgroup into LDS and then lives in registers.  Mapping:
//   - a lane owns one PAIR of adjacent blocks (36 B, two dwordx4 + one dword
//     load), i.e. 64 consecutive activations, for R rows at a time;
//   - L lanes cover one row (L = next power of two >= pairs per row, <= 64),
//     so a wave's load instruction reads 64/L consecutive rows = contiguous
//     bytes;
//   - all R x 9 dword loads of a wave are issued before the first use, so a
//     wave keeps R*2304 bytes in flight;
//   - the L partial sums of a row are combined with DPP adds.
#include "q4_0_mfma.hpp"

namespace {

constexpr int kThreads = 512;
constexpr int kWaves = kThreads / LEV_WAVE;

// Resident workgroups per CU the persistent grid is sized for (tunable for
// experiments through LEV_Q4_WG_PER_CU).
uint32_t lev_q4_gemv_wg_per_cu() {
    static uint32_t v = [] {
        const char *e = getenv("LEV_Q4_WG_PER_CU");
        int n = e ? atoi(e) : 0;
        return (uint32_t)(n > 0 && n <= 16 ? n : 2);
    }();
    return v;
}

// Loads the R pairs a lane owns in the tile whose first row is `row0`.
// Branch-free: lanes past the end of the row or of the matrix read a valid
// pair from a clamped address; they multiply it by zero activations or
// never store the result.
template <int L, int R>
__device__ __forceinline__ void load_tile(const uint8_t *__restrict__ w, uint64_t row_bytes,
                                          uint32_t row0, uint32_t rows, uint32_t pairs, uint32_t p,
                                          uint32_t D[R][9]) {
    constexpr int G = LEV_WAVE / L;
    const uint32_t pc = p < pairs ? p : pairs - 1u;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        uint32_t row = row0 + r * G;
        lev_q4_load_pair(w + (row < rows ? row : rows - 1u) * row_bytes + (uint64_t)pc * 36u, D[r]);
    }
}

// Multiplies a tile and leaves the finished dot products of the workgroup's
// kWaves*G*R rows in ysh; the first threads then store them contiguously.
template <int L, int R, bool MULTI>
__device__ __forceinline__ void finish_tile(const uint8_t *__restrict__ w, uint64_t row_bytes,
                                            const lev_f32x4 *xs, const float *bsum, float *ysh,
                                            float *__restrict__ y, uint32_t tile_base,
                                            uint32_t in_tile, uint32_t rows, uint32_t pairs,
                                            uint32_t lp, const lev_q4_pair_x &px0,
                                            const uint32_t D[R][9]) {
    constexpr int G = LEV_WAVE / L;
    constexpr uint32_t kRowsPerTile = kWaves * G * R;
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = lev_q4_pair_dot(D[r], px0);

    if (MULTI) {
        // Rows longer than 64 pairs: further column chunks of the same rows.
        for (uint32_t c = LEV_WAVE; c < pairs; c += LEV_WAVE) {
            const uint32_t p = c + lp;
            uint32_t E[R][9];
            load_tile<L, R>(w, row_bytes, tile_base + in_tile, rows, pairs, p, E);
            lev_q4_pair_x px;
            lev_q4_fetch_x_sums(xs, bsum, pairs, p < pairs ? p : pairs - 1u, px);
            const float keep = p < pairs ? 1.0f : 0.0f;   // partial last chunk
#pragma unroll
            for (int r = 0; r < R; ++r) acc[r] = fmaf(keep, lev_q4_pair_dot(E[r], px), acc[r]);
        }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
        float s = lev_group_sum<L>(acc[r]);
        if (lp == L - 1) ysh[in_tile + r * G] = s;
    }
    lev_barrier_lds();
    if (threadIdx.x < kRowsPerTile && tile_base + threadIdx.x < rows)
        y[tile_base + threadIdx.x] = ysh[threadIdx.x];
    lev_barrier_lds();   // ysh is reused by the next tile
}

// One tile per workgroup, straight-line code: used whenever the whole matrix
// fits in one resident wave of workgroups (every decode-sized matrix).  EXACT
// means pairs == L and pairs*16 == NS*kThreads: no padding lanes, no bounds
// tests, so the compiler can wait for each weight load separately and start
// multiplying as soon as the first one lands.
template <int L, int R, int NS, bool EXACT>
__global__ void __launch_bounds__(kThreads)
q4_0_gemv_tile(const uint8_t *__restrict__ w, const float *__restrict__ x, float *__restrict__ y,
               uint32_t pairs, uint32_t rows) {
    extern __shared__ lev_f32x4 xs[];
    constexpr int G = LEV_WAVE / L;
    constexpr uint32_t kRowsPerTile = kWaves * G * R;
    __shared__ float ysh[kRowsPerTile];
    float *bsum = reinterpret_cast<float *>(xs + 16u * (pairs + 1u));
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & (LEV_WAVE - 1);
    const uint32_t wave = tid / LEV_WAVE;
    const uint32_t grp = lane / L;
    const uint32_t lp = lane % L;
    const uint64_t row_bytes = (uint64_t)pairs * 36u;
    const uint32_t in_tile = wave * (G * R) + grp;
    const uint32_t base = blockIdx.x * kRowsPerTile;

    lev_f32x4 xv[NS];
    lev_q4_stage_x_load<NS, EXACT>(x, pairs, tid, kThreads, xv);
    uint32_t D[R][9];
    load_tile<L, R>(w, row_bytes, base + in_tile, rows, pairs, lp, D);
    lev_q4_stage_x_store_sums<NS, EXACT>(x, xs, bsum, pairs, tid, kThreads, xv);
    lev_barrier_lds();

    lev_q4_pair_x px;
    const bool p_ok = EXACT || lp < pairs;
    lev_q4_fetch_x_sums(xs, bsum, pairs, p_ok ? lp : pairs - 1u, px);
    if (!EXACT) {
#pragma unroll
        for (int q = 0; q < 16; ++q) px.xr[q] = p_ok ? px.xr[q] : lev_f32x4{0.f, 0.f, 0.f, 0.f};
        px.sum_a = p_ok ? px.sum_a : 0.f;
        px.sum_b = p_ok ? px.sum_b : 0.f;
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
        float s = lev_group_sum<L>(lev_q4_pair_dot(D[r], px));
        if (lp == L - 1) ysh[in_tile + r * G] = s;
    }
    lev_barrier_lds();
    if (tid < kRowsPerTile && base + tid < rows) y[base + tid] = ysh[tid];
}

// Workgroups of 8 waves walk tiles of kWaves*G*R rows with a stride of
// gridDim.x tiles, double-buffering the weight registers so that the loads
// of tile t+1 are in flight while tile t is being multiplied.
template <int L, int R, bool MULTI, int NS>
__global__ void __launch_bounds__(kThreads)
q4_0_gemv_pairs(const uint8_t *__restrict__ w, const float *__restrict__ x, float *__restrict__ y,
                uint32_t pairs, uint32_t rows) {
    extern __shared__ lev_f32x4 xs[];
    constexpr int G = LEV_WAVE / L;                 // rows per wave-wide load
    constexpr uint32_t kRowsPerTile = kWaves * G * R;
    __shared__ float ysh[kRowsPerTile];
    float *bsum = reinterpret_cast<float *>(xs + 16u * (pairs + 1u));
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & (LEV_WAVE - 1);
    const uint32_t wave = tid / LEV_WAVE;
    const uint32_t grp = lane / L;
    const uint32_t lp = lane % L;
    const bool p_ok = lp < pairs;
    const uint64_t row_bytes = (uint64_t)pairs * 36u;
    const uint32_t in_tile = wave * (G * R) + grp;   // rows of one wave are wave*(G*R) + r*G + grp
    const uint32_t step = gridDim.x * kRowsPerTile;

    uint32_t base = blockIdx.x * kRowsPerTile;
    if (base >= rows) return;

    // Activations first (16 KB, L2 hits after the first workgroup), then the
    // first tile's weights: the activations are staged and fetched while the
    // weights are still in flight.
    lev_f32x4 xv[NS];
    lev_q4_stage_x_load<NS>(x, pairs, tid, kThreads, xv);
    uint32_t Da[R][9], Db[R][9];
    load_tile<L, R>(w, row_bytes, base + in_tile, rows, pairs, lp, Da);
    lev_q4_stage_x_store_sums<NS>(x, xs, bsum, pairs, tid, kThreads, xv);
    lev_barrier_lds();

    // Activations of the lane's first pair stay in registers for every tile;
    // lanes past the end of the row hold zeros.
    lev_q4_pair_x px0;
    lev_q4_fetch_x_sums(xs, bsum, pairs, p_ok ? lp : pairs - 1u, px0);
#pragma unroll
    for (int q = 0; q < 16; ++q) px0.xr[q] = p_ok ? px0.xr[q] : lev_f32x4{0.f, 0.f, 0.f, 0.f};
    px0.sum_a = p_ok ? px0.sum_a : 0.f;
    px0.sum_b = p_ok ? px0.sum_b : 0.f;

    if (step >= rows) {   // the grid covers every tile once: nothing to prefetch
        finish_tile<L, R, MULTI>(w, row_bytes, xs, bsum, ysh, y, base, in_tile, rows, pairs, lp, px0, Da);
        return;
    }
    // The prefetch is unconditional (past the last tile it re-reads the last
    // row, which is harmless): a branch around it would make the compiler
    // wait for the prefetched data before the current tile is multiplied.
    while (true) {
        uint32_t next = base + step;
        load_tile<L, R>(w, row_bytes, next + in_tile, rows, pairs, lp, Db);
        finish_tile<L, R, MULTI>(w, row_bytes, xs, bsum, ysh, y, base, in_tile, rows, pairs, lp, px0, Da);
        if (next >= rows) break;
        base = next;
        next = base + step;
        load_tile<L, R>(w, row_bytes, next + in_tile, rows, pairs, lp, Da);
        finish_tile<L, R, MULTI>(w, row_bytes, xs, bsum, ysh, y, base, in_tile, rows, pairs, lp, px0, Db);
        if (next >= rows) break;
        base = next;
    }
}

// Any geometry (odd block counts, rows that are only 2-byte aligned, rows too
// long for LDS): one wave per row, 16-bit loads, activations from global
// memory.  Correct everywhere, fast nowhere; the pair kernel covers every
// shape the models on this path use.
__global__ void __launch_bounds__(256)
q4_0_gemv_generic(const uint8_t *__restrict__ w, const float *__restrict__ x,
                  float *__restrict__ y, uint32_t blocks_per_row, uint32_t rows) {
    const uint32_t lane = threadIdx.x & (LEV_WAVE - 1);
    const uint32_t row = blockIdx.x * 4u + threadIdx.x / LEV_WAVE;
    if (row >= rows) return;
    const uint8_t *rp = w + (uint64_t)row * blocks_per_row * 18u;
    float acc = 0.f;
    for (uint32_t b = lane; b < blocks_per_row; b += LEV_WAVE) {
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
    if (lane == LEV_WAVE - 1) y[row] = acc;
}

// NS = float4 of the activation vector each thread stages from registers.
template <int L, int R, bool MULTI = false, int NS = 1>
hipError_t launch_pairs(lev_ctx *ctx, const uint8_t *w, const float *x, float *y, uint32_t pairs,
                        uint32_t rows, int persistent = -1) {
    constexpr uint32_t rows_per_tile = kWaves * (LEV_WAVE / L) * R;
    uint32_t blocks = (rows + rows_per_tile - 1) / rows_per_tile;
    // built-in choice (persistent < 0): one workgroup per tile while every tile is resident at once
    const bool tiles = persistent < 0 ? blocks <= (uint32_t)ctx->num_cus * 4u : persistent == 0;
    if (!MULTI && tiles) {
        // every tile is resident at once: one straight-line tile per workgroup
        size_t lds1 = (size_t)16 * (pairs + 1) * sizeof(lev_f32x4) + (size_t)2 * pairs * sizeof(float);
        const bool exact = pairs == (uint32_t)L && pairs * 16u == (uint32_t)NS * kThreads;
        if (exact)
            hipLaunchKernelGGL((q4_0_gemv_tile<L, R, NS, true>), dim3(blocks), dim3(kThreads), lds1,
                               ctx->stream, w, x, y, pairs, rows);
        else
            hipLaunchKernelGGL((q4_0_gemv_tile<L, R, NS, false>), dim3(blocks), dim3(kThreads), lds1,
                               ctx->stream, w, x, y, pairs, rows);
        return hipGetLastError();
    }
    // Persistent grid: as many workgroups as stay resident at once.
    uint32_t cap = (uint32_t)ctx->num_cus * lev_q4_gemv_wg_per_cu();
    if (blocks > cap) blocks = cap;
    size_t lds = (size_t)16 * (pairs + 1) * sizeof(lev_f32x4) + (size_t)2 * pairs * sizeof(float);
    if (lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&q4_0_gemv_pairs<L, R, MULTI, NS>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL((q4_0_gemv_pairs<L, R, MULTI, NS>), dim3(blocks), dim3(kThreads), lds, ctx->stream, w, x,
                       y, pairs, rows);
    return hipGetLastError();
}

}  // namespace

bool lev_q4_0_mfma_gemv_usable(const uint8_t *w, const float *x, uint32_t in_dim);
hipError_t lev_q4_0_mfma_gemv_launch(lev_ctx *ctx, const uint8_t *w, const float *x, float *y, uint32_t in_dim,
                                     uint32_t rows, int persistent);

// Enqueue without argument checks (callers validated the geometry).
hipError_t lev_q4_0_gemv_launch(lev_ctx *ctx, const uint8_t *w, const float *x, float *y,
                                uint32_t in_dim, uint32_t rows) {
    const uint32_t nb = in_dim / 32u;
    {
        // a schedule installed for this shape (lev_hip_forge_select) overrides the built-in choice
        const lev_schedule *sel = lev_selected(ctx, LEV_OP_Q4_0_GEMV, in_dim, rows, 1);
        static const int env_mfma = [] {
            const char *e = getenv("LEV_Q4_MFMA");   // experiments: 0 = vector-ALU kernels, 1 = matrix-core kernel
            return e ? atoi(e) : -1;
        }();
        const bool usable = lev_q4_0_mfma_gemv_usable(w, x, in_dim);
        if (usable && (sel ? sel->family == 1u : env_mfma != 0))
            return lev_q4_0_mfma_gemv_launch(ctx, w, x, y, in_dim, rows, sel ? (int)sel->persistent : -1);
    }
    const bool pairable = (nb % 2u == 0u) && ((reinterpret_cast<uintptr_t>(w) & 3u) == 0u) &&
                          (in_dim <= 32768u) && ((reinterpret_cast<uintptr_t>(x) & 15u) == 0u);
    if (!pairable) {
        uint32_t blocks = (rows + 3u) / 4u;
        hipLaunchKernelGGL(q4_0_gemv_generic, dim3(blocks), dim3(256), 0, ctx->stream, w, x, y,
                           nb, rows);
        return hipGetLastError();
    }
    const uint32_t pairs = nb / 2u;
    // a schedule installed for this shape (lev_hip_forge_select) overrides the built-in choice
    const lev_schedule *sel = lev_selected(ctx, LEV_OP_Q4_0_GEMV, in_dim, rows, 1);
    if (sel && pairs > 16 && pairs <= 64) {
        const int pm = (int)sel->persistent;
        if (pairs > 32) {
            if (sel->rows_in_flight == 1) return launch_pairs<64, 1, false, 2>(ctx, w, x, y, pairs, rows, pm);
            if (sel->rows_in_flight == 2) return launch_pairs<64, 2, false, 2>(ctx, w, x, y, pairs, rows, pm);
            return launch_pairs<64, 4, false, 2>(ctx, w, x, y, pairs, rows, pm);
        }
        if (sel->rows_in_flight == 1) return launch_pairs<32, 1>(ctx, w, x, y, pairs, rows, pm);
        if (sel->rows_in_flight == 2) return launch_pairs<32, 2>(ctx, w, x, y, pairs, rows, pm);
        return launch_pairs<32, 4>(ctx, w, x, y, pairs, rows, pm);
    }
    if (pairs > 32) {
        if (pairs > 64) return launch_pairs<64, 2, true, 4>(ctx, w, x, y, pairs, rows);
        // One row per wave and pass measured fastest at 4096 and 32768 rows:
        // 100 VGPRs leave five waves per SIMD to hide the HBM latency.
        return launch_pairs<64, 1, false, 2>(ctx, w, x, y, pairs, rows);
    }
    if (pairs > 16) return launch_pairs<32, 4>(ctx, w, x, y, pairs, rows);
    if (pairs > 8) return launch_pairs<16, 4>(ctx, w, x, y, pairs, rows);
    if (pairs > 4) return launch_pairs<8, 4>(ctx, w, x, y, pairs, rows);
    return launch_pairs<4, 4>(ctx, w, x, y, pairs, rows);
}

// The candidate schedules of a Q4_0 GEMV shape, the built-in choice first
// (Q4ScheduleDeriver.derive, Q4Lowering.swift:283-362: baseline first, then the
// legal variants, bounded).  Shapes outside the two widest kernel families have
// the built-in choice only.
uint32_t lev_q4_0_gemv_candidates(const lev_ctx *ctx, uint32_t in_dim, uint32_t rows, lev_schedule *out,
                                  uint32_t capacity) {
    const uint32_t nb = in_dim / 32u, pairs = nb / 2u;
    const bool family = (nb % 2u == 0u) && in_dim <= 32768u && pairs > 16 && pairs <= 64;
    const uint32_t base_r = pairs > 32 ? 1u : 4u;
    const uint32_t lanes = pairs > 32 ? 64u : 32u;
    auto is_persistent = [&](uint32_t r) {
        const uint32_t rows_per_tile = kWaves * (LEV_WAVE / lanes) * r;
        return (rows + rows_per_tile - 1) / rows_per_tile > (uint32_t)ctx->num_cus * 4u ? 1u : 0u;
    };
    lev_schedule all[12];
    uint32_t n = 0;
    auto push = [&](uint32_t r, uint32_t p) {
        for (uint32_t i = 0; i < n; ++i)
            if (all[i].family == 0u && all[i].rows_in_flight == r && all[i].persistent == p) return;
        all[n++] = lev_schedule{LEV_OP_Q4_0_GEMV, 0u, r, p};
    };
    // rows of whole 256-value tasks: the matrix-core kernel (family 1), the built-in choice, with
    // one workgroup per round of row groups or a resident grid
    if (in_dim % 256u == 0u && in_dim <= kLevQ4MfmaMaxInDim) {
        const uint32_t ntask = in_dim >> 8, slots = ntask <= 16u ? 16u / ntask : 1u;
        const uint32_t nrounds = ((rows + 15u) / 16u + slots - 1u) / slots;
        const uint32_t builtin = nrounds <= (uint32_t)ctx->num_cus ? 0u : 1u;
        all[n++] = lev_schedule{LEV_OP_Q4_0_GEMV, 1u, 0u, builtin};
        all[n++] = lev_schedule{LEV_OP_Q4_0_GEMV, 1u, 0u, 1u - builtin};
    }
    if (!family) {
        push(0u, 0u);   // the vector-ALU kernel of the shape, which has no parameters here
    } else {
        push(base_r, is_persistent(base_r));
        for (uint32_t r : {1u, 2u, 4u})
            for (uint32_t p : {0u, 1u}) push(r, p);
    }
    for (uint32_t i = 0; i < n && i < capacity; ++i) out[i] = all[i];
    return n;
}

extern "C" int lev_hip_q4_0_gemv(lev_ctx *ctx, const void *d_w, size_t w_bytes, uint64_t w_off,
                                 const float *d_x, size_t x_count, float *d_y, size_t y_capacity,
                                 uint32_t in_dim, uint32_t out_rows) {
    LEV_REQUIRE_CTX(ctx);
    lev_geom g;
    int st = lev_check_matvec(ctx, "q4_0_gemv", 32, 18, d_w, w_bytes, w_off, d_x, x_count, in_dim,
                              d_y, y_capacity, out_rows, in_dim, out_rows, &g);
    if (st != LEV_OK) return st;
    const uint8_t *w = static_cast<const uint8_t *>(d_w) + w_off;
    return lev_hip_check(ctx, lev_q4_0_gemv_launch(ctx, w, d_x, d_y, in_dim, out_rows),
                         "q4_0_gemv launch");
}

// Shared host + device helpers of the gfx950 quantized-matmul library.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "../../include/leviathan_hip.h"

// ---------------------------------------------------------------------------
// context
// ---------------------------------------------------------------------------

struct lev_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    bool owns_stream = false;
    hipDeviceProp_t props{};
    int num_cus = 0;
    std::string last_error;
    // Engine-owned scratch (the reference sizes its MoE scratch once and keeps
    // it, Gemma4.swift:2025-2059).  Grown on demand, never shrunk.
    void *scratch = nullptr;
    size_t scratch_bytes = 0;
    // Recorded programs keep the scratch address they were recorded with.  While
    // any program is alive a buffer that has to make room for a larger one is
    // parked here instead of freed, so replaying the program stays valid; the
    // parked buffers go when the last program or the context is destroyed.
    int live_programs = 0;
    std::vector<void *> retired_scratch;
    // Device-side error flag written by kernels that validate device-resident
    // arguments (expert ids); read back by lev_hip_sync.
    // Per-workgroup (best, second, index) partials of the greedy-token epilogue
    // of the Q6_K GEMV: fixed size, allocated with the context and never moved,
    // so a recorded GEMV needs no grow-on-demand scratch.
    void *argmax_partials = nullptr;
    static constexpr uint32_t kArgmaxPartials = 4096;   // entries of 16 bytes
    // word 0: error flags raised by kernels (read and cleared by lev_hip_sync);
    // words kTicketWord..+3: arrival counters of the router kernel, one per token,
    // zero between launches (the last workgroup to arrive resets its counter)
    int *d_flag = nullptr;
    // words kArgmaxTicketWord + 1024*k, k = 0..8: arrival counters of the greedy-token merge
    // (4 KB apart: counters that share a cache line serialise in one L2 channel), zero between launches
    static constexpr uint32_t kFlagWords = 10 * 1024, kTicketWord = 16, kArgmaxTicketWord = 1024;
    int *h_flag = nullptr;   // pinned
    // True between lev_hip_program_begin and lev_hip_program_end: the stream
    // is being captured, so nothing may allocate or synchronise.
    bool recording = false;
    // Schedules installed per (op, shape) by lev_hip_forge_select; the matvec
    // entry points look their shape up here before their built-in choice.
    struct selection {
        uint32_t in_dim, rows, ncol;
        lev_schedule schedule;
    };
    std::vector<selection> selections;
    // Device address, on this context's GPU, of the static scratch array of
    // lev_hip_moe_layer_q4_0_noalloc (looked up once at context creation).
    void *moe_static_scratch = nullptr;
};

// Looks the static MoE scratch array up on the current device (moe.hip).
int lev_moe_static_scratch_init(lev_ctx *ctx);

// The schedule installed for this op and shape, or nullptr.
const lev_schedule *lev_selected(const lev_ctx *ctx, uint32_t op, uint32_t in_dim, uint32_t rows, uint32_t ncol);

int lev_fail(lev_ctx *ctx, int status, const char *fmt, ...);
int lev_hip_check(lev_ctx *ctx, hipError_t err, const char *what);
// Returns device scratch of at least `bytes` (256-byte aligned) or nullptr.
void *lev_scratch(lev_ctx *ctx, size_t bytes);
// Zero-fills `bytes` (a multiple of 4) with a small kernel on the context's
// stream (safe to record into a HIP graph, unlike a memset node).
hipError_t lev_zero_async(lev_ctx *ctx, void *d_ptr, size_t bytes);

#define LEV_REQUIRE_CTX(ctx)                         \
    do {                                             \
        if (!(ctx)) return LEV_ERR_INVALID_ARGUMENT; \
    } while (0)

#define LEV_HIP(ctx, expr)                                      \
    do {                                                        \
        int _st = lev_hip_check((ctx), (expr), #expr);          \
        if (_st != LEV_OK) return _st;                          \
    } while (0)

// Geometry shared by every quantized matvec: dims, block multiple, workload
// caps, weight extent inside [w_off, w_bytes), x count, y capacity.
// Order of checks follows Q4.swift:168-193 and Gemma4.swift:2599-2627.
struct lev_geom {
    uint64_t blocks_per_row;
    uint64_t row_bytes;
    uint64_t weight_bytes;
};
int lev_check_matvec(lev_ctx *ctx, const char *op, uint32_t block_values, uint32_t block_bytes,
                     const void *d_w, size_t w_bytes, uint64_t w_off, const void *d_x,
                     size_t x_count, uint64_t x_needed, const void *d_y, size_t y_capacity,
                     uint64_t y_needed, uint64_t in_dim, uint64_t out_rows, lev_geom *g);

// ---------------------------------------------------------------------------
// device helpers
// ---------------------------------------------------------------------------

#define LEV_WAVE 64

typedef uint32_t lev_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t lev_u32x2 __attribute__((ext_vector_type(2)));
typedef float lev_f32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 lev_f16x2 __attribute__((ext_vector_type(2)));

// Loads that only promise the alignment the GGUF block layouts give
// (Q4_0 and Q6_K blocks are 2-byte aligned; pairs of Q4_0 blocks 4-byte).
struct __attribute__((packed, aligned(4))) lev_u32x4_a4 { uint32_t v[4]; };
struct __attribute__((packed, aligned(4))) lev_u32_a4 { uint32_t v; };
struct __attribute__((packed, aligned(4))) lev_u32x2_a4 { uint32_t v[2]; };
struct __attribute__((packed, aligned(2))) lev_u32_a2 { uint32_t v; };
struct __attribute__((packed, aligned(2))) lev_u16_a2 { uint16_t v; };

__device__ __forceinline__ float lev_f16_bits_to_f32(uint32_t bits16) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)bits16);
}

// Sum over the 64 lanes of a wave with DPP (no LDS traffic); every lane of
// the last row-of-16 ends with partial results, lane 63 with the total.
template <int CTRL, int ROW_MASK = 0xF, bool BOUND = true>
__device__ __forceinline__ float lev_dpp_add(float v) {
    int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xF, BOUND);
    return v + __builtin_bit_cast(float, moved);
}

// Sum across groups of L consecutive lanes (L a power of two <= 64).  On
// return lane (group_base + L - 1)... holds no special role: every lane of
// the group holds the group's sum for L <= 16; for L = 32 / 64 use the value
// from lane L-1 of the group (highest lane).
template <int L>
__device__ __forceinline__ float lev_group_sum(float v) {
    if (L >= 2) v = lev_dpp_add<0xB1>(v);    // quad_perm [1,0,3,2]
    if (L >= 4) v = lev_dpp_add<0x4E>(v);    // quad_perm [2,3,0,1]
    if (L >= 8) v = lev_dpp_add<0x141>(v);   // row_half_mirror
    if (L >= 16) v = lev_dpp_add<0x140>(v);  // row_mirror
    if (L >= 32) v = lev_dpp_add<0x142, 0xA, false>(v);  // row_bcast:15 -> rows 1,3
    if (L >= 64) v = lev_dpp_add<0x143, 0xC, false>(v);  // row_bcast:31 -> rows 2,3
    return v;
}

// The same in f64 (two DPP moves and one add per step).  For L <= 16 every lane
// of a group ends with the group's sum; for L = 32 / 64 read the highest lane.
template <int CTRL, int ROW_MASK = 0xF, bool BOUND = true>
__device__ __forceinline__ double lev_dpp_add_f64(double v) {
    const int lo = __builtin_amdgcn_update_dpp(0, __double2loint(v), CTRL, ROW_MASK, 0xF, BOUND);
    const int hi = __builtin_amdgcn_update_dpp(0, __double2hiint(v), CTRL, ROW_MASK, 0xF, BOUND);
    return v + __hiloint2double(hi, lo);
}

template <int L>
__device__ __forceinline__ double lev_group_sum_f64(double v) {
    if (L >= 2) v = lev_dpp_add_f64<0xB1>(v);
    if (L >= 4) v = lev_dpp_add_f64<0x4E>(v);
    if (L >= 8) v = lev_dpp_add_f64<0x141>(v);
    if (L >= 16) v = lev_dpp_add_f64<0x140>(v);
    if (L >= 32) v = lev_dpp_add_f64<0x142, 0xA, false>(v);
    if (L >= 64) v = lev_dpp_add_f64<0x143, 0xC, false>(v);
    return v;
}

__device__ __forceinline__ float lev_wave_sum_broadcast(float v) {
    v = lev_group_sum<64>(v);
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

// Workgroup barrier that orders LDS traffic only: it waits for this wave's LDS
// operations and leaves its global loads in flight.  __syncthreads() carries a
// workgroup fence for which the compiler drains every outstanding load first,
// i.e. the prefetch of the next tile: inside a streaming loop that turns every
// iteration into a full memory round trip.
__device__ __forceinline__ void lev_barrier_lds() {
    __builtin_amdgcn_s_waitcnt(0xC07F);   // lgkmcnt(0); vmcnt and expcnt left open
    asm volatile("s_barrier" ::: "memory");
}

// ---- shared by the kernels in which a wave owns one column block of the matrix (a Q4_0 task,
// a Q4_K or Q6_K superblock column) and `wpr` waves of a workgroup of 16 cover a row ----

// Sum over lanes l, l ^ 16, l ^ 32, l ^ 48 (the four lane groups of a matrix-core row), in every
// lane, in f64, by two row swaps per dword: no LDS.
__device__ __forceinline__ double lev_row_sum_f64(double v) {
    uint32_t lo = (uint32_t)__double2loint(v), hi = (uint32_t)__double2hiint(v);
    auto a0 = __builtin_amdgcn_permlane32_swap(lo, lo, false, false);
    auto a1 = __builtin_amdgcn_permlane32_swap(hi, hi, false, false);
    v = __hiloint2double((int)a1[0], (int)a0[0]) + __hiloint2double((int)a1[1], (int)a0[1]);
    lo = (uint32_t)__double2loint(v);
    hi = (uint32_t)__double2hiint(v);
    a0 = __builtin_amdgcn_permlane16_swap(lo, lo, false, false);
    a1 = __builtin_amdgcn_permlane16_swap(hi, hi, false, false);
    return __hiloint2double((int)a1[0], (int)a0[0]) + __hiloint2double((int)a1[1], (int)a0[1]);
}

// Largest of an unsigned value over the 16 lanes of a row of the wave, in every lane of the row:
// quad swaps, then the two row mirrors (DPP: no LDS, no other unit).  Magnitudes of floats
// compare as their bit patterns do; NaN and infinity sort above every number.
__device__ __forceinline__ uint32_t lev_row16_max_u32(uint32_t v) {
#define LEV_ROW16_MAX_STEP(CTRL)                                                                        \
    {                                                                                                   \
        const uint32_t o = (uint32_t)__builtin_amdgcn_update_dpp((int)v, (int)v, CTRL, 0xF, 0xF, false); \
        v = o > v ? o : v;                                                                              \
    }
    LEV_ROW16_MAX_STEP(0xB1)    // quad_perm [1,0,3,2]
    LEV_ROW16_MAX_STEP(0x4E)    // quad_perm [2,3,0,1]
    LEV_ROW16_MAX_STEP(0x141)   // row_half_mirror
    LEV_ROW16_MAX_STEP(0x140)   // row_mirror
#undef LEV_ROW16_MAX_STEP
    return v;
}

// The same over all 64 lanes: the four rows' maxima meet by two row swaps.
__device__ __forceinline__ uint32_t lev_wave_max_u32(uint32_t v) {
    v = lev_row16_max_u32(v);
    const auto s0 = __builtin_amdgcn_permlane32_swap(v, v, false, false);
    v = s0[0] > s0[1] ? s0[0] : s0[1];
    const auto s1 = __builtin_amdgcn_permlane16_swap(v, v, false, false);
    return s1[0] > s1[1] ? s1[0] : s1[1];
}

// Four values per lane whose sums over lanes l, l ^ 16, l ^ 32, l ^ 48 are wanted: lane group
// g = lane / 16 gets the sum of v[g], by two exchanges between the halves of the wave and one
// between the rows of a half (three swaps for four sums; the additions pair the lane groups as
// lev_row_sum_f64 does: (g, g ^ 2) first, then (g, g ^ 1)).
__device__ __forceinline__ float lev_lanegroup_sums4(const float v[4]) {
    const auto s02 = __builtin_amdgcn_permlane32_swap(__float_as_uint(v[0]), __float_as_uint(v[2]), false, false);
    const auto s13 = __builtin_amdgcn_permlane32_swap(__float_as_uint(v[1]), __float_as_uint(v[3]), false, false);
    const float a = __uint_as_float(s02[0]) + __uint_as_float(s02[1]);
    const float b = __uint_as_float(s13[0]) + __uint_as_float(s13[1]);
    const auto sab = __builtin_amdgcn_permlane16_swap(__float_as_uint(a), __float_as_uint(b), false, false);
    return __uint_as_float(sab[0]) + __uint_as_float(sab[1]);
}

// Keeps a value that the tail of a round needs (an LDS offset, an output pointer, a mask)
// computed where it is written: between the load requests and the first wait, where
// instructions cost nothing.  Left to itself the compiler sinks such arithmetic to its use,
// behind the barrier, where every instruction is on the critical path of the launch.
template <typename T>
__device__ __forceinline__ void lev_pin(T &v) {
    asm volatile("" : "+v"(v));
}

// wave -> (slot, position in the slot) as 4-bit entries of two 64-bit kernel arguments, for 16
// waves of which `wpr` (1..16) share a group of rows: a division in front of a kernel's first
// load would cost some thirty instructions.  Waves beyond the last whole slot get slot 15 or the
// first unused one (>= 16 / wpr): idle.
inline void lev_wave_tables(uint32_t wpr, uint64_t *slot_of_wave, uint64_t *pos_of_wave) {
    *slot_of_wave = 0;
    *pos_of_wave = 0;
    for (uint32_t wv = 0; wv < 16u; ++wv) {
        *slot_of_wave |= (uint64_t)(wv / wpr > 15u ? 15u : wv / wpr) << (4u * wv);
        *pos_of_wave |= (uint64_t)(wv % wpr) << (4u * wv);
    }
}

// Hand-over of a few words from one workgroup to whichever workgroup arrives last at a
// counter, WITHOUT a release fence (on this chip a device-scope release writes back every
// dirty line of the XCD's L2, the kernel's own outputs included).  The order is kept by three
// properties of gfx942 / gfx950 hardware, not by the HIP memory model, so the code that uses
// it is compiled for these targets only:
//   1. a relaxed agent-scope atomic store is a store with sc1 set: it is written through the
//      XCD's L2 to memory, and its completion is counted in vmcnt;
//   2. `s_waitcnt vmcnt(0)` therefore returns only once those stores have reached memory; the
//      relaxed agent-scope fetch_add that follows is issued after it (the asm statement is a
//      compiler barrier for memory operations as well);
//   3. a relaxed agent-scope atomic load is a load with sc1 set: it is served from memory, not
//      from a line the reader's own L2 may still hold.
// The last arriver sees the final count only after every other workgroup's stores completed.
#if defined(__HIP_DEVICE_COMPILE__) && !defined(__gfx950__) && !defined(__gfx942__)
#error "lev_publish_wait relies on gfx942/gfx950 store completion (vmcnt) and sc1 write-through semantics"
#endif
__device__ __forceinline__ void lev_publish_wait() {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// Overflow-safe tanh and gelu_tanh(g)*u exactly as the reference kernels
// spell them (g4_tanh / g4_gelu_up_value, Gemma4.swift:4364-4377).
__device__ __forceinline__ float lev_stable_tanh(float x) {
    float e = __expf(-2.0f * fabsf(x));
    return copysignf((1.0f - e) / (1.0f + e), x);
}

__device__ __forceinline__ float lev_gelu_up_value(float g, float u) {
    float inner = 0.7978845608028654f * (g + 0.044715f * g * g * g);
    float gelu = 0.5f * g * (1.0f + lev_stable_tanh(inner));
    return gelu * u;
}

// Running top two of a stream of logits (value, second value, index of the best):
// the state of the greedy-token epilogue (argmax + margin, lev-forge/src/ops.rs:479-516).
#pragma once

#include "lev_common.hpp"

namespace {

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


// Top two over the 64 lanes of a wave, in every lane.  Inside a row of 16 lanes the partner's
// record comes by DPP, across rows by a row swap: no LDS traffic, a third of the latency of six
// rounds of lane permutations.  (top2_merge gives the same record whichever side is "mine".)
__device__ __forceinline__ top2 top2_wave(top2 m) {
#define LEV_TOP2_DPP(CTRL)                                                                                         \
    {                                                                                                              \
        top2 o;                                                                                                    \
        o.best = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, m.best),            \
                                                                       __builtin_bit_cast(int, m.best), CTRL, 0xF, \
                                                                       0xF, false));                               \
        o.second = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, m.second),        \
                                                                         __builtin_bit_cast(int, m.second), CTRL,  \
                                                                         0xF, 0xF, false));                        \
        o.idx = (uint32_t)__builtin_amdgcn_update_dpp((int)m.idx, (int)m.idx, CTRL, 0xF, 0xF, false);              \
        m = top2_merge(m, o);                                                                                      \
    }
    LEV_TOP2_DPP(0xB1)    // quad_perm [1,0,3,2]
    LEV_TOP2_DPP(0x4E)    // quad_perm [2,3,0,1]
    LEV_TOP2_DPP(0x141)   // row_half_mirror
    LEV_TOP2_DPP(0x140)   // row_mirror: the 16 lanes of a row hold the row's record
#undef LEV_TOP2_DPP
    {
        const auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(m.best), __float_as_uint(m.best), false, false);
        const auto s2 = __builtin_amdgcn_permlane32_swap(__float_as_uint(m.second), __float_as_uint(m.second), false, false);
        const auto ix = __builtin_amdgcn_permlane32_swap(m.idx, m.idx, false, false);
        m = top2_merge(top2{__uint_as_float(b[0]), __uint_as_float(s2[0]), ix[0]},
                       top2{__uint_as_float(b[1]), __uint_as_float(s2[1]), ix[1]});
    }
    {
        const auto b = __builtin_amdgcn_permlane16_swap(__float_as_uint(m.best), __float_as_uint(m.best), false, false);
        const auto s2 = __builtin_amdgcn_permlane16_swap(__float_as_uint(m.second), __float_as_uint(m.second), false, false);
        const auto ix = __builtin_amdgcn_permlane16_swap(m.idx, m.idx, false, false);
        m = top2_merge(top2{__uint_as_float(b[0]), __uint_as_float(s2[0]), ix[0]},
                       top2{__uint_as_float(b[1]), __uint_as_float(s2[1]), ix[1]});
    }
    return m;
}

constexpr float kTop2Floor = -INFINITY;

}  // namespace

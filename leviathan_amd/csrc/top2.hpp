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

}  // namespace

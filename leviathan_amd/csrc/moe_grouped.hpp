// Interface between the MoE entry points and the many-token (grouped,
// matrix-core) expert path.
#pragma once

#include "lev_common.hpp"

struct lev_moe_grouped_args {
    const uint8_t *base;
    uint64_t gate_off, up_off, down_off;
    uint64_t gate_stride, up_stride, down_stride;
    uint32_t hidden, inter, experts, top_k, tokens;
};

// A work item of the integer matrix-core kernels: `count` (1..8) pairs of one expert, the pairs
// `first ..` of the expert-ordered list.  pair[k] is the (token * top_k + slot) index of column k,
// src[k] its token; columns past `count` repeat the last.
struct alignas(16) lev_grp_item {
    int32_t expert, count, first, pad;
    int32_t pair[8], src[8];
};

// Where a workgroup of the integer matrix-core kernels starts: its stretch of the line of rounds
// and the header of the first item it touches (one load in front of the first weight request
// instead of three that depend on each other).
struct alignas(32) lev_grp_start {
    uint32_t first_round, end_round, item;
    int32_t expert, count;
    uint32_t pad[3];
};

size_t lev_moe_grouped_scratch_bytes(const lev_moe_grouped_args &a);
// Geometry the grouped path serves (the caller also checks 4-byte aligned pools).
bool lev_moe_grouped_usable(const lev_ctx *ctx, const lev_moe_grouped_args &a);
// act: f32 [tokens*top_k][inter] (written here, read by the down stage).
hipError_t lev_moe_grouped_launch(lev_ctx *ctx, const lev_moe_grouped_args &a, const float *x,
                                  const int32_t *ids, const float *weights, float *y, float *act,
                                  void *scratch);

// Schedule candidates and per-shape selection for the matvec operators.
//
// The reference derives candidate schedules from the operation's shape and the
// device, runs and gates every candidate and keeps a measured selection
// (lev-forge/src/schedule.rs:83-105, lev-cli/src/main.rs:1977-2022,
// Q4Lowering.swift:283-362).  Its candidates are emitted shader sources; here
// they are the precompiled kernel variants of this library.  This file holds
// the part that lives in the library: the candidate lists and the table the
// entry points consult.  Running, gating and timing the candidates is host
// work above the C ABI.
#include "lev_common.hpp"

uint32_t lev_q4_0_gemv_candidates(const lev_ctx *ctx, uint32_t in_dim, uint32_t rows, lev_schedule *out,
                                  uint32_t capacity);
uint32_t lev_q4_k_gemv_candidates(const lev_ctx *ctx, uint32_t in_dim, uint32_t rows, uint32_t ncol,
                                  lev_schedule *out, uint32_t capacity);
uint32_t lev_q4_k_gemv_q8_candidates(const lev_ctx *ctx, uint32_t in_dim, uint32_t rows, uint32_t ncol,
                                     lev_schedule *out, uint32_t capacity);
uint32_t lev_q6_k_gemv_candidates(const lev_ctx *ctx, uint32_t in_dim, uint32_t rows, lev_schedule *out,
                                  uint32_t capacity);
uint32_t lev_q6_k_gemv_q8_candidates(const lev_ctx *ctx, uint32_t in_dim, uint32_t rows, uint32_t ncol,
                                     lev_schedule *out, uint32_t capacity);
uint32_t lev_moe_layer_candidates(const lev_ctx *ctx, uint32_t hidden, uint32_t inter, uint32_t tokens,
                                  lev_schedule *out, uint32_t capacity);

const lev_schedule *lev_selected(const lev_ctx *ctx, uint32_t op, uint32_t in_dim, uint32_t rows, uint32_t ncol) {
    for (const lev_ctx::selection &s : ctx->selections)
        if (s.schedule.op == op && s.in_dim == in_dim && s.rows == rows && s.ncol == ncol) return &s.schedule;
    return nullptr;
}

namespace {

constexpr uint32_t kMaxCandidates = 16;

int shape_ok(lev_ctx *ctx, uint32_t op, uint32_t in_dim, uint32_t rows, uint32_t ncol) {
    if (op < LEV_OP_Q4_0_GEMV || op > LEV_OP_MOE_LAYER_Q4_0)
        return lev_fail(ctx, LEV_ERR_INVALID_ARGUMENT, "forge: unknown op %u", op);
    const bool moe = op == LEV_OP_MOE_LAYER_Q4_0;
    const uint32_t block = op == LEV_OP_Q4_0_GEMV || moe ? 32u : 256u;
    if (in_dim == 0 || rows == 0 || in_dim % block != 0 || (moe && rows % block != 0) ||
        in_dim > LEV_MAX_Q4_INPUT_DIM || rows > LEV_MAX_Q4_OUTPUT_DIM)
        return lev_fail(ctx, LEV_ERR_BAD_DIMENSIONS, "forge: %u x %u is not a shape of this op", rows, in_dim);
    const bool one_column = op == LEV_OP_Q4_0_GEMV || op == LEV_OP_Q6_K_GEMV;
    if (ncol == 0 || ncol > (moe ? 4u : (uint32_t)LEV_MAX_GEMV_COLUMNS) || (one_column && ncol != 1))
        return lev_fail(ctx, LEV_ERR_BAD_DIMENSIONS, "forge: %u columns", ncol);
    return LEV_OK;
}

uint32_t candidates(const lev_ctx *ctx, uint32_t op, uint32_t in_dim, uint32_t rows, uint32_t ncol,
                    lev_schedule *out, uint32_t capacity) {
    if (op == LEV_OP_Q4_0_GEMV) return lev_q4_0_gemv_candidates(ctx, in_dim, rows, out, capacity);
    if (op == LEV_OP_Q4_K_GEMV) return lev_q4_k_gemv_candidates(ctx, in_dim, rows, ncol, out, capacity);
    if (op == LEV_OP_Q6_K_GEMV) return lev_q6_k_gemv_candidates(ctx, in_dim, rows, out, capacity);
    if (op == LEV_OP_Q6_K_GEMV_Q8) return lev_q6_k_gemv_q8_candidates(ctx, in_dim, rows, ncol, out, capacity);
    if (op == LEV_OP_MOE_LAYER_Q4_0) return lev_moe_layer_candidates(ctx, in_dim, rows, ncol, out, capacity);
    return lev_q4_k_gemv_q8_candidates(ctx, in_dim, rows, ncol, out, capacity);
}

}  // namespace

extern "C" int lev_hip_forge_candidates(lev_ctx *ctx, uint32_t op, uint32_t in_dim, uint32_t rows, uint32_t ncol,
                                        lev_schedule *out, uint32_t capacity, uint32_t *count) {
    LEV_REQUIRE_CTX(ctx);
    if (!count || (!out && capacity)) return lev_fail(ctx, LEV_ERR_INVALID_ARGUMENT, "forge_candidates: null pointer");
    int st = shape_ok(ctx, op, in_dim, rows, ncol);
    if (st != LEV_OK) return st;
    *count = candidates(ctx, op, in_dim, rows, ncol, out, capacity);
    return LEV_OK;
}

extern "C" int lev_hip_forge_select(lev_ctx *ctx, uint32_t in_dim, uint32_t rows, uint32_t ncol,
                                    const lev_schedule *schedule) {
    LEV_REQUIRE_CTX(ctx);
    if (!schedule) return lev_fail(ctx, LEV_ERR_INVALID_ARGUMENT, "forge_select: null schedule");
    int st = shape_ok(ctx, schedule->op, in_dim, rows, ncol);
    if (st != LEV_OK) return st;
    lev_schedule legal[kMaxCandidates];
    uint32_t n = candidates(ctx, schedule->op, in_dim, rows, ncol, legal, kMaxCandidates);
    if (n > kMaxCandidates) n = kMaxCandidates;
    bool found = false;
    for (uint32_t i = 0; i < n; ++i)
        found = found || (legal[i].family == schedule->family && legal[i].rows_in_flight == schedule->rows_in_flight &&
                          legal[i].persistent == schedule->persistent);
    if (!found)
        return lev_fail(ctx, LEV_ERR_INVALID_ARGUMENT,
                        "forge_select: schedule (family %u, rows in flight %u, persistent %u) is not a candidate "
                        "of op %u at %u x %u x %u", schedule->family, schedule->rows_in_flight,
                        schedule->persistent, schedule->op, rows, in_dim, ncol);
    for (lev_ctx::selection &s : ctx->selections)
        if (s.schedule.op == schedule->op && s.in_dim == in_dim && s.rows == rows && s.ncol == ncol) {
            s.schedule = *schedule;
            return LEV_OK;
        }
    ctx->selections.push_back(lev_ctx::selection{in_dim, rows, ncol, *schedule});
    return LEV_OK;
}

extern "C" int lev_hip_forge_clear(lev_ctx *ctx, uint32_t op, uint32_t in_dim, uint32_t rows, uint32_t ncol) {
    LEV_REQUIRE_CTX(ctx);
    for (size_t i = 0; i < ctx->selections.size(); ++i) {
        const lev_ctx::selection &s = ctx->selections[i];
        if (s.schedule.op == op && s.in_dim == in_dim && s.rows == rows && s.ncol == ncol) {
            ctx->selections.erase(ctx->selections.begin() + (long)i);
            break;
        }
    }
    return LEV_OK;
}

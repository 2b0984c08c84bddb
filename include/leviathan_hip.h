/*
 * leviathan_hip.h -- C ABI of the MI355X (gfx950) quantized-matmul library.
 *
 * This is the surface LeviathanCore's Swift operator API (or the Rust
 * Builder) binds instead of Metal / Vulkan.  The reference has no FFI of its
 * own for this path, so every entry point cites the reference operator it
 * stands in for (paths relative to the dhihm/leviathan tree).
 *
 * Conventions
 *   - plain C: opaque context, raw pointers, sizes; no exceptions cross the
 *     boundary.  Every call returns a lev_status; lev_hip_last_error() gives
 *     the text of the last failure on that context.
 *   - pointers named d_* are DEVICE pointers (from lev_hip_buf_alloc or any
 *     other HIP allocation of the same process, e.g. a torch tensor).
 *   - operators are ENQUEUED on the context's stream and return immediately
 *     (the reference's "deferred segment", Gemma4.swift:2313-2376); call
 *     lev_hip_sync() before reading results on the host.
 *   - all geometry / extent / overflow checks run on the host before any
 *     launch; a failed check launches nothing (fail closed, Q4.swift:168-210,
 *     Gemma4.swift:2599-2627).
 *   - a context is not thread-safe (Gemma4Runner is a non-Sendable class).
 *   - weights stay exactly as stored in the GGUF file; nothing is repacked.
 */
#ifndef LEVIATHAN_HIP_H
#define LEVIATHAN_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Mirrors Q4Error (Sources/LeviathanCore/Q4.swift:17-31). */
typedef enum lev_status {
    LEV_OK = 0,
    LEV_ERR_BAD_DIMENSIONS = 1,
    LEV_ERR_WRONG_INPUT_COUNT = 2,
    LEV_ERR_NON_FINITE_INPUT = 3,
    LEV_ERR_NON_FINITE_SCALE = 4,
    LEV_ERR_NON_FINITE_OUTPUT = 5,
    LEV_ERR_EXCEEDS_MODEL_WORKLOAD = 6,
    LEV_ERR_INTEGER_OVERFLOW = 7,
    LEV_ERR_DEVICE_UNAVAILABLE = 8,      /* metalUnavailable */
    LEV_ERR_KERNEL_LOAD_FAILED = 9,      /* shaderCompileFailed */
    LEV_ERR_FUNCTION_MISSING = 10,
    LEV_ERR_COMMAND_FAILED = 11,         /* commandBufferFailed */
    LEV_ERR_EXCEEDS_MAX_BUFFER_LENGTH = 12,
    LEV_ERR_EXCEEDS_WORKING_SET = 13,    /* exceedsRecommendedWorkingSet */
    LEV_ERR_INVALID_ARGUMENT = 14        /* null pointer / misuse of this ABI */
} lev_status;

/* GGMLTensorType (Sources/LeviathanCore/GGUF.swift:58-91) and
 * GgmlType (rust/crates/lev-gguf/src/lib.rs:94-112): GGML type ids. */
typedef enum lev_qtype {
    LEV_TYPE_F32 = 0,
    LEV_TYPE_F16 = 1,
    LEV_TYPE_Q4_0 = 2,
    LEV_TYPE_Q4_K = 12,
    LEV_TYPE_Q6_K = 14
} lev_qtype;

/* ModelWorkloadLimits (Sources/LeviathanCore/Q4.swift:8-15). */
#define LEV_MAX_Q4_INPUT_DIM (1 << 22)
#define LEV_MAX_Q4_OUTPUT_DIM (1 << 22)
#define LEV_MAX_Q4_WEIGHT_BYTES ((uint64_t)32 << 30)

/* Largest column count of the multi-column GEMV (nb in q8.rs:196-326). */
#define LEV_MAX_GEMV_COLUMNS 16

typedef struct lev_ctx lev_ctx;

/* Q4MatvecEvidence (Sources/LeviathanCore/Q4.swift:116-123). */
typedef struct lev_evidence {
    char device_name[128];
    uint64_t device_max_buffer_length;
    uint64_t recommended_max_working_set_size;
    int64_t out_dim;
    int64_t in_dim;
    char command_status[32];
} lev_evidence;

/* ---- library ---- */

/* ABI version of this header (bumped on any signature change; 2: without lev_hip_prefetch, Q4_0 GEMV
 * schedules of family 1, MoE schedules with `persistent`). */
int lev_hip_abi_version(void);
const char *lev_hip_status_name(int status);

/* ---- context: device + one stream (MTLDevice + MTLCommandQueue,
 * Gemma4.swift:518-524; VulkanContext::open, lev-vulkan/src/lib.rs) ----
 * `stream` is the hipStream_t to enqueue on; NULL is HIP's default (null)
 * stream.  Pass LEV_HIP_OWN_STREAM for a stream the context creates and owns. */
#define LEV_HIP_OWN_STREAM ((void *)(intptr_t)-1)
int lev_hip_ctx_create(int device, void *stream, lev_ctx **out);
int lev_hip_ctx_destroy(lev_ctx *ctx);
/* flushOpenSegment / cmd.waitUntilCompleted (Gemma4.swift:2313, 2465-2468). */
int lev_hip_sync(lev_ctx *ctx);
const char *lev_hip_last_error(lev_ctx *ctx);
int lev_hip_device_name(lev_ctx *ctx, char *out, size_t cap);

/* ---- recorded programs: record once, replay (Program / Step,
 * rust/crates/lev-vulkan/src/engine.rs:94-141; deferred segments,
 * Gemma4.swift:2313-2376) ----
 * Between begin and end every operator call on the context is recorded
 * instead of executed; run() replays the whole sequence with one submission.
 * The context must own its stream or sit on a non-default stream.  Pointers
 * and sizes are frozen into the program, the context's scratch address
 * included.  Scratch is never grown while recording (run each MoE shape once
 * before recording it; a call that would have to grow it fails with
 * LEV_ERR_EXCEEDS_WORKING_SET and records nothing).  An eager call after
 * recording may still grow the scratch: the buffer a live program was recorded
 * with then stays allocated until the last program of the context is
 * destroyed, so replaying stays valid. */
typedef struct lev_program lev_program;
int lev_hip_program_begin(lev_ctx *ctx);
int lev_hip_program_end(lev_ctx *ctx, lev_program **out);
int lev_hip_program_run(lev_ctx *ctx, lev_program *program);
int lev_hip_program_destroy(lev_ctx *ctx, lev_program *program);
int lev_hip_program_node_count(lev_program *program, size_t *out);

/* ---- buffers (device.makeBuffer, Q4.swift:223-231; Buf, engine.rs:10-40) ---- */
int lev_hip_buf_alloc(lev_ctx *ctx, size_t bytes, void **d_out);
int lev_hip_buf_free(lev_ctx *ctx, void *d_ptr);
int lev_hip_buf_upload(lev_ctx *ctx, void *d_dst, const void *host_src, size_t bytes);
int lev_hip_buf_download(lev_ctx *ctx, void *host_dst, const void *d_src, size_t bytes);

/* ---- measurement helpers (lev vk-bw, rust/crates/lev-cli/src/main.rs:1876-1935) ----
 * One pass of 128-bit reads over `bytes` bytes (result discarded): the
 * streaming-read ceiling of the device.  workgroups == 0 picks a default. */
int lev_hip_stream_read_probe(lev_ctx *ctx, const void *d_src, size_t bytes, uint32_t *d_sink,
                              uint32_t workgroups);
/* Enqueues a kernel that does nothing: the launch-to-launch floor. */
int lev_hip_empty_launch(lev_ctx *ctx);

/* ---- dequantise (decodeBlock, Q4.swift:54; Q6.swift:23; dequant_block_f32,
 * lev-cpu/src/lib.rs:111): nblocks blocks of `type` -> f32, bit-exact ---- */
int lev_hip_dequant(lev_ctx *ctx, int type, const void *d_w, size_t w_bytes, uint64_t w_off,
                    uint64_t nblocks, float *d_out, size_t out_capacity);

/* ---- decode GEMV, y = W x ----
 * Kernel ABI (uint2 p=(inDim,outRows), ulong wOff, uchar* wbase, float* x,
 * float* y): Gemma4.swift:3931-3936; operator matvec / matvecDispatch,
 * Gemma4.swift:2583, 2638.  w_bytes is the extent of the weight buffer,
 * w_off the byte offset of the tensor (or expert slice) inside it. */
int lev_hip_q4_0_gemv(lev_ctx *ctx, const void *d_w, size_t w_bytes, uint64_t w_off,
                      const float *d_x, size_t x_count, float *d_y, size_t y_capacity,
                      uint32_t in_dim, uint32_t out_rows);

/* Q6_K GEMV (g4_q6_matvec, Gemma4.swift:4065; q6k.matvec, lev-forge/src/q6k.rs:61)
 * with the greedy-token epilogue fused behind it (argmax, lev-forge/src/ops.rs:479-516):
 * d_argmax / d_margin may be NULL to skip it.  Lowest index wins ties;
 * margin = best - second best. */
int lev_hip_q6_k_gemv(lev_ctx *ctx, const void *d_w, size_t w_bytes, uint64_t w_off,
                      const float *d_x, size_t x_count, float *d_y, size_t y_capacity,
                      uint32_t in_dim, uint32_t out_rows, uint32_t *d_argmax, float *d_margin);

/* Q4_K multi-column GEMV for MTP verify (Builder::matvec, lev-model/src/gpu.rs:334-370;
 * q4k.matvec nb columns, lev-forge/src/glsl.rs:157-281) with the RMSNorm of
 * the input fused in front (Builder::norm_quant, gpu.rs:295; rmsnorm,
 * lev-model/src/lib.rs:110-114).  x is [ncol][in_dim], y is [ncol][rows]
 * (y[col*rows + row], glsl.rs:247).  d_gain == NULL skips the norm.
 * Five to eight columns of in_dim <= 4096 keep ncol*in_dim*4 bytes (+ 1 KB) of
 * digit planes in the context's scratch between two kernels; while a program is
 * being recorded and the scratch is still smaller than that, a kernel that needs
 * none runs instead (same results), so the call never fails for want of scratch. */
int lev_hip_q4_k_gemv_ncol(lev_ctx *ctx, const void *d_w, size_t w_bytes, uint64_t w_off,
                           const float *d_x, size_t x_count, const float *d_gain, float eps,
                           float *d_y, size_t y_capacity, uint32_t in_dim, uint32_t rows,
                           uint32_t ncol);

/* Q6_K multi-column GEMV on f32 activations: the LM head (or any Q6_K tensor) applied to
 * ncol columns per weight read, as Builder::matvec does for Q4_K
 * (lev-model/src/gpu.rs:334-370; single-column q6k.matvec, lev-forge/src/q6k.rs:61-187),
 * with the same optional RMSNorm in front (d_gain == NULL skips it).  Same layouts as
 * lev_hip_q4_k_gemv_ncol: x is [ncol][in_dim], y[col*rows + row].  Sums are formed
 * without rounding, so a column's result does not depend on ncol.  Weights 2-byte
 * aligned (GGUF), x and gain 16-byte aligned, in_dim a multiple of 256 and no wider
 * than the activation staging of the matrix-core kernel holds in LDS (16384 on MI355X,
 * never beyond 32768): wider rows are
 * refused with LEV_ERR_EXCEEDS_MODEL_WORKLOAD and nothing is launched; lev_hip_q6_k_gemv
 * takes them a column at a time. */
int lev_hip_q6_k_gemv_ncol(lev_ctx *ctx, const void *d_w, size_t w_bytes, uint64_t w_off,
                           const float *d_x, size_t x_count, const float *d_gain, float eps,
                           float *d_y, size_t y_capacity, uint32_t in_dim, uint32_t rows,
                           uint32_t ncol);

/* ---- int8-activation decode path ----
 * Activation quantiser: groups of 32, d = amax/127, q = roundEven(v * 127/amax),
 * s = d * sum(q) (quantize_q8, lev-cpu/src/lib.rs:295-322; emit_quantize,
 * lev-forge/src/q8.rs:20-51), optionally behind the residual add and the
 * RMSNorm of the block input (emit_norm_quant, q8.rs:127-164; Builder::norm_quant,
 * lev-model/src/gpu.rs:295):
 *   d_add  != NULL: x += add first, written back to d_x (read-write then);
 *   d_gain != NULL: v = rmsnorm(x, eps) * gain (f64 mean of squares as the
 *                   reference CPU path, lev-model/src/lib.rs:110-114), else v = x;
 *   d_y    != NULL: v is also stored as f32.
 * x is [ncol][n], n a multiple of 32.  d_xq: int8 [ncol][n] (4-byte aligned),
 * d_xs: f32 pairs (d, s) [ncol][n/32]. */
int lev_hip_norm_quant_q8(lev_ctx *ctx, float *d_x, size_t x_count, const float *d_add,
                          const float *d_gain, float eps, int8_t *d_xq, float *d_xs, float *d_y,
                          uint32_t n, uint32_t ncol);

/* Q4_K GEMV on the int8 activations above, ncol columns per weight read
 * (q4k.q8.matvec, emit_q4k_q8, lev-forge/src/q8.rs:191-326; oracle
 * matvec_q4k_q8_f64, lev-cpu/src/lib.rs:324-331).  Integer dot products per
 * sub-block are exact; y[col*rows + row].  x_count counts int8 codes
 * (in_dim * ncol); weights, d_xq and d_xs 16-byte aligned. */
int lev_hip_q4_k_gemv_q8(lev_ctx *ctx, const void *d_w, size_t w_bytes, uint64_t w_off,
                         const int8_t *d_xq, const float *d_xs, size_t x_count, float *d_y,
                         size_t y_capacity, uint32_t in_dim, uint32_t rows, uint32_t ncol);

/* Q6_K GEMV on the same int8 activations (q6k.q8.matvec, emit_q6k_q8,
 * lev-forge/src/q8.rs:330-447; oracle matvec_q6k_q8_f64, lev-cpu/src/lib.rs:333-337):
 * the LM head of a multi-column verify step.  Weights 2-byte aligned (GGUF). */
int lev_hip_q6_k_gemv_q8(lev_ctx *ctx, const void *d_w, size_t w_bytes, uint64_t w_off,
                         const int8_t *d_xq, const float *d_xs, size_t x_count, float *d_y,
                         size_t y_capacity, uint32_t in_dim, uint32_t rows, uint32_t ncol);

/* act = silu(gate) * up fused with the quantiser (emit_swiglu_quant,
 * lev-forge/src/q8.rs:166-177; Builder::swiglu_quant, lev-model/src/gpu.rs:322-330).
 * count values (a multiple of 32); d_act (optional) also receives act as f32. */
int lev_hip_swiglu_quant_q8(lev_ctx *ctx, const float *d_gate, const float *d_up, size_t count,
                            int8_t *d_xq, float *d_xs, float *d_act);

/* ---- prefill GEMM (Builder::matvec_rows with gemm, gpu.rs:345-355;
 * q4k gemm blocked, lev-forge/src/coopmat.rs:236-323) ----
 * x is fp16 [tokens][in_dim], y is f32 [tokens][rows]; W is dequantised to
 * fp16 tiles in LDS and multiplied on the matrix cores, f32 accumulate.
 * in_dim at most 4194304, tokens at most 1048576 (LEV_ERR_BAD_DIMENSIONS beyond). */
int lev_hip_q4_k_gemm_prefill(lev_ctx *ctx, const void *d_w, size_t w_bytes, uint64_t w_off,
                              const uint16_t *d_x_f16, size_t x_count, float *d_y,
                              size_t y_capacity, uint32_t in_dim, uint32_t rows,
                              uint32_t tokens);
/* The same for Q6_K weights (q6k gemm blocked, lev-forge/src/coopmat.rs:333-425):
 * W is dequantised to fp16 as (d*sc)*(q-32) in f32, rounded to nearest even.
 * Weights 2-byte aligned (GGUF), x 16-byte aligned. */
int lev_hip_q6_k_gemm_prefill(lev_ctx *ctx, const void *d_w, size_t w_bytes, uint64_t w_off,
                              const uint16_t *d_x_f16, size_t x_count, float *d_y,
                              size_t y_capacity, uint32_t in_dim, uint32_t rows,
                              uint32_t tokens);
/* act_f16 (lev-forge/src/coopmat.rs:49): f32 -> f16, round to nearest even. */
int lev_hip_f32_to_f16(lev_ctx *ctx, const float *d_x, uint16_t *d_out, size_t n);

/* Embedding lookup from a Q4_K table (embed_q4k, lev-forge/src/ops.rs:523-555; Builder step
 * "embed", lev-model/src/gpu.rs:457): column c of out (dim floats) is row d_tokens[c] of the
 * [vocab][dim] table, dequantised bit-exactly as lev_hip_dequant does.  A token id >= vocab
 * writes nothing and is reported by the next lev_hip_sync as LEV_ERR_BAD_DIMENSIONS. */
int lev_hip_embed_q4_k(lev_ctx *ctx, const void *d_w, size_t w_bytes, uint64_t w_off,
                       const uint32_t *d_tokens, uint32_t ntokens, float *d_out, size_t out_capacity,
                       uint32_t dim, uint32_t vocab);

/* ---- elementwise operators of the runner ---- */
/* rmsnorm(x:y:n:vectors:weightTensor:) (Gemma4.swift:3014; kernel :4247);
 * d_weight may be NULL (scale-free). */
int lev_hip_rmsnorm(lev_ctx *ctx, const float *d_x, float *d_y, uint32_t n, uint32_t vectors,
                    const float *d_weight, float eps);
/* geluUp(gu:y:n:) (Gemma4.swift:3103; kernel :4380): y[i] = gelu_tanh(gu[i]) * gu[n+i]. */
int lev_hip_gelu_up(lev_ctx *ctx, const float *d_gu, float *d_y, uint32_t n);
/* axpy(x:xOffset:y:c:n:) (Gemma4.swift:3115; kernel :4459): y += c * x. */
int lev_hip_axpy(lev_ctx *ctx, const float *d_x, float *d_y, float c, uint32_t n);
/* argmax step (lev-forge/src/ops.rs:479-516): per column of `vocab` logits. */
int lev_hip_argmax(lev_ctx *ctx, const float *d_logits, uint32_t vocab, uint32_t ncol,
                   uint32_t *d_index, float *d_margin);

/* ---- MoE ---- */
/* Router: F32 matvec (g4_f32_matvec, Gemma4.swift:4160) then softmax in f64,
 * top-k with ties to the lower index, renormalise, times the per-expert
 * scale (Gemma4.swift:3795-3810).  x [tokens][hidden], router weights
 * [experts][hidden]; outputs ids i32 [tokens][top_k], weights f32
 * [tokens][top_k]; d_scores (optional) f32 [tokens][experts];
 * d_expert_scale may be NULL (== 1). */
int lev_hip_moe_route_topk(lev_ctx *ctx, const float *d_router_w, const float *d_x,
                           const float *d_expert_scale, int32_t *d_ids, float *d_weights,
                           float *d_scores, uint32_t hidden, uint32_t experts, uint32_t top_k,
                           uint32_t tokens);

/* Expert weight pools in Q4_0.  Expert e's gate rows start at
 * gate_off + e*gate_stride (same for up, down): MoEModelBinding.offsets,
 * MoEModelBinding.swift:174-214, 284-292.  The reference's fused gate|up
 * tensor [2I, H] is described by up_off = gate_off + I*(H/32)*18 and
 * up_stride = gate_stride. */
typedef struct lev_moe_experts {
    const void *d_base;      /* weight buffer holding all three pools */
    size_t base_bytes;       /* its extent */
    uint64_t gate_off, up_off, down_off;
    uint64_t gate_stride, up_stride, down_stride;
    uint32_t hidden, inter, experts;
} lev_moe_experts;

/* Routed experts: for each token, for each slot in order,
 * y += w_slot * W_down[e] * (gelu_tanh(W_gate[e] x) * (W_up[e] x))
 * (runMoeBatchedRouted, Gemma4.swift:2073; per-slot loop :3856-3880;
 * moesimd_gu / moesimd_dn, MoESIMDLowering.swift:497-636).  y is
 * overwritten (the accumulator reset of Gemma4.swift:3841 is included).
 * ids must be distinct per token and < experts (checked on the device;
 * a violation is reported by the next lev_hip_sync as LEV_ERR_BAD_DIMENSIONS).
 * d_act (optional) receives the activations [tokens][top_k][inter]. */
int lev_hip_moe_experts_q4_0(lev_ctx *ctx, const lev_moe_experts *pools, const float *d_x,
                             const int32_t *d_ids, const float *d_weights, float *d_y,
                             float *d_act, uint32_t top_k, uint32_t tokens);

/* Whole layer: route + experts in one enqueue (forwardLayer MoE block,
 * Gemma4.swift:3795-3880, without the Gemma-specific input scaling). */
int lev_hip_moe_layer_q4_0(lev_ctx *ctx, const lev_moe_experts *pools, const float *d_router_w,
                           const float *d_expert_scale, const float *d_x, float *d_y,
                           int32_t *d_ids, float *d_weights, uint32_t top_k, uint32_t tokens);

/* The same block for callers that cannot allocate device memory: code that is
 * being captured into a HIP graph, tight serving loops, harnesses that forbid
 * hipMalloc.  NO COUNTERPART IN THE REFERENCE (its MoE scratch is sized once by
 * the engine, Gemma4.swift:2025-2059); it exists for those callers only.
 * Arguments and results are those of lev_hip_moe_layer_q4_0, bit for bit; the
 * router scores and the expert activations live in a static device array of
 * LEV_NOALLOC_MOE_SCRATCH_BYTES that every GPU holds until the process ends,
 * and the call itself allocates nothing.  Limits: tokens <=
 * LEV_NOALLOC_MOE_MAX_TOKENS and 256-byte-rounded
 * tokens*experts*4 + tokens*top_k*inter*4 <= LEV_NOALLOC_MOE_SCRATCH_BYTES,
 * otherwise LEV_ERR_EXCEEDS_WORKING_SET and nothing is launched.  All calls on
 * one GPU share the one array: calls that overlap in time on the same GPU
 * (from two contexts or streams) race. */
#define LEV_NOALLOC_MOE_SCRATCH_BYTES (1u << 20)
#define LEV_NOALLOC_MOE_MAX_TOKENS 4u
int lev_hip_moe_layer_q4_0_noalloc(lev_ctx *ctx, const lev_moe_experts *pools,
                                   const float *d_router_w, const float *d_expert_scale,
                                   const float *d_x, float *d_y, int32_t *d_ids, float *d_weights,
                                   uint32_t top_k, uint32_t tokens);

/* ---- host-array convenience twins of the standalone backends ----
 * Q4MetalBackend.matvecReporting (Q4.swift:165-269) and
 * Q6MetalBackend.matvecReporting (Q6.swift:199-285): validate, upload,
 * run, download, re-check the output is finite, report evidence. */
int lev_hip_q4_0_matvec_reporting(const uint8_t *blocks, size_t blocks_count, int64_t out_dim,
                                  int64_t in_dim, const float *x, size_t x_count, float *y_out,
                                  lev_evidence *evidence);
int lev_hip_q6_k_matvec_reporting(const uint8_t *blocks, size_t blocks_count, int64_t out_dim,
                                  int64_t in_dim, const float *x, size_t x_count, float *y_out,
                                  lev_evidence *evidence);

/* ---- schedule candidates and per-shape selection (the library side of the
 * forge loop: schedule::derive, lev-forge/src/schedule.rs:83-105;
 * Q4ScheduleDeriver.derive, Q4Lowering.swift:283-362; the measured selection
 * of lev-cli/src/main.rs:1977-2022 runs above this ABI) ----
 * The reference derives schedules and emits a shader per candidate; here a
 * schedule names one of the precompiled kernel variants.  Candidate 0 is
 * always the built-in choice (the reference's BASELINE).  A selection applies
 * to exactly one (op, in_dim, rows, ncol) on this context and is consulted by
 * the operator's entry point before its built-in choice.  The Q6_K head and the
 * MoE layer have candidates as the reference's own forges do (vk_q6k,
 * lev-cli/src/main.rs:467 and lev-forge/src/q6k.rs:175; MoELoweringForge.forge,
 * MoELowering.swift:1896-1985).  For LEV_OP_MOE_LAYER_Q4_0 the shape is
 * (in_dim = hidden, rows = expert intermediate size, ncol = tokens, 1..4). */
#define LEV_OP_Q4_0_GEMV 1u
#define LEV_OP_Q4_K_GEMV 2u
#define LEV_OP_Q4_K_GEMV_Q8 3u
#define LEV_OP_Q6_K_GEMV 4u
#define LEV_OP_Q6_K_GEMV_Q8 5u
#define LEV_OP_MOE_LAYER_Q4_0 6u
typedef struct lev_schedule {
    uint32_t op;             /* LEV_OP_* */
    uint32_t family;         /* Q4_K: 1 = matrix-core kernel, 0 = vector-ALU (int8: dot4) kernel; Q4_0: 1 = integer
                                matrix-core kernel (rows of whole 256-value tasks up to 8192 wide), 0 = vector-ALU kernels;
                                Q6_K: 2 = integer matrix-core kernel, 0 = digit-plane dot4 kernel (both exact),
                                1 = one wave per row with f64 sums;
                                Q6_K x int8: 1 = integer matrix-core kernel, 0 = dot4 kernel; MoE layer: who selects the experts: 1 = the gate/up workgroups
                                themselves, 2 = the last workgroup of the router kernel to finish, 0 = a top-k
                                kernel of its own ahead of them */
    uint32_t rows_in_flight; /* Q4_0 family 0: rows a wave keeps in flight (1, 2, 4; 0 = no variants for the shape);
                                Q6_K: waves that share a row (family 0: 1, 2) or a group of 16 rows (family 2:
                                2, 4, 8, 16; 0 = a wave per superblock column, for rows up to 4096 wide);
                                Q6_K x int8: columns per pass over the
                                weights; MoE layer: gate/up workgroups aimed at per CU (1, 2, 4) */
    uint32_t persistent;     /* Q4_0, Q6_K x int8: 0 = one workgroup per row tile, 1 = resident grid walking
                                the tiles; MoE layer: 0 = expert kernels on the integer matrix cores where the
                                shape allows, 1 = vector-ALU expert kernels */
} lev_schedule;
/* Writes min(*count, capacity) candidates; *count is the full number. */
int lev_hip_forge_candidates(lev_ctx *ctx, uint32_t op, uint32_t in_dim, uint32_t rows,
                             uint32_t ncol, lev_schedule *out, uint32_t capacity, uint32_t *count);
/* Installs `schedule` (which must be one of the shape's candidates, else
 * LEV_ERR_INVALID_ARGUMENT) for the shape; replaces an earlier selection. */
int lev_hip_forge_select(lev_ctx *ctx, uint32_t in_dim, uint32_t rows, uint32_t ncol,
                         const lev_schedule *schedule);
/* Back to the built-in choice for the shape. */
int lev_hip_forge_clear(lev_ctx *ctx, uint32_t op, uint32_t in_dim, uint32_t rows, uint32_t ncol);

#ifdef __cplusplus
}
#endif
#endif /* LEVIATHAN_HIP_H */

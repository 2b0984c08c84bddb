/*
 * lev_oracle.h -- CPU restatement of Leviathan's quantized-matmul hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library links, loads or
 * calls this code: it exists so that tests, the smoke check and the
 * benchmark's CPU-baseline leg can compare the HIP kernels against the
 * reference's own CPU arithmetic on identical inputs.
 *
 * Every function names the reference source it restates (paths are relative
 * to the dhihm/leviathan tree).  The reference is Swift and Rust; neither
 * toolchain exists in this build environment, so the reference itself is not
 * compiled.  Each restated function is pinned by the reference's own
 * known-answer tests (see tests/test_oracle_*.py, which cite them).
 *
 * Parity status of every function in this file:
 *   pinned by reference known-answer vectors, closed forms or brute force:
 *     f16 conversions, SplitMix64, Q4_0 / Q6_K / Q4_K decode and matvecs,
 *     int8 activation quantisation, RMSNorm, GELU-tanh*up, stable tanh,
 *     argmax + margin, normalised error metric, MoE expert composite,
 *     prefill GEMM oracle definition.
 *   pinned by source text + invariants + brute force + library cross-check
 *   only (the reference holds no unit test for it):
 *     router softmax / top-k / renormalise (levo_router_topk).
 *
 * All f32 arithmetic is compiled with -ffp-contract=off so that sums follow
 * the source order of the reference with no fused multiply-add.
 */
#ifndef LEV_ORACLE_H
#define LEV_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Status codes: same numbering as lev_status in include/leviathan_hip.h,
 * which in turn mirrors Q4Error (Sources/LeviathanCore/Q4.swift:17-31). */
enum {
    LEVO_OK = 0,
    LEVO_BAD_DIMENSIONS = 1,
    LEVO_WRONG_INPUT_COUNT = 2,
    LEVO_NON_FINITE_INPUT = 3,
    LEVO_NON_FINITE_SCALE = 4,
    LEVO_NON_FINITE_OUTPUT = 5,
    LEVO_EXCEEDS_MODEL_WORKLOAD = 6,
    LEVO_INTEGER_OVERFLOW = 7,
    LEVO_INVALID_ARGUMENT = 14
};

#define LEVO_Q4_0_BLOCK_BYTES 18
#define LEVO_Q4_0_BLOCK_VALUES 32
#define LEVO_Q4_K_BLOCK_BYTES 144
#define LEVO_Q6_K_BLOCK_BYTES 210
#define LEVO_QK_K 256

/* ---- half precision (rust/crates/lev-cpu/src/lib.rs:14-60) ---- */
double levo_f16_to_f64(uint16_t h);
float levo_f16_to_f32(uint16_t h);
uint16_t levo_f32_to_f16_bits(float v);

/* ---- SplitMix64 (Sources/LeviathanCore/RNG.swift:4-24,
 *                  rust/crates/lev-cpu/src/lib.rs:357-373) ---- */
uint64_t levo_splitmix64_next(uint64_t *state);
float levo_next_uniform(uint64_t *state);      /* Swift nextUniform  */
float levo_next_signed_unit(uint64_t *state);  /* Rust next_signed_unit */
void levo_fill_uniform(uint64_t seed, float *out, size_t n);      /* seededInput */
void levo_fill_signed_unit(uint64_t seed, float *out, size_t n);

/* ---- Q4_0 (Sources/LeviathanCore/Q4.swift:33-113) ---- */
int levo_q4_0_decode_block(const uint8_t *block, float *out32);
int levo_q4_0_dequant(const uint8_t *w, size_t nblocks, float *out);
/* Q4_0.matvecReference: f32, block-local partial then ascending blocks. */
int levo_q4_0_matvec_ref(const uint8_t *w, size_t w_bytes, int64_t out_dim,
                         int64_t in_dim, const float *x, size_t x_count, float *y);
/* Same arithmetic, rows split over `threads` host threads (the way the
 * reference's CPU forward runs matvecs, rust/crates/lev-model/src/lib.rs:184-199). */
int levo_q4_0_matvec_ref_mt(const uint8_t *w, size_t w_bytes, int64_t out_dim,
                            int64_t in_dim, const float *x, size_t x_count, float *y,
                            int threads);
/* The serial GPU kernel's summation order (leviathan_q4_matvec,
 * Sources/LeviathanCore/Q4.swift:139-161): straight into the row sum,
 * low/high nibble interleaved. */
int levo_q4_0_matvec_kernel_order(const uint8_t *w, size_t w_bytes, int64_t out_dim,
                                  int64_t in_dim, const float *x, size_t x_count, float *y);
/* Q4Oracle.matvecFP64 (Sources/LeviathanCore/Q4Lowering.swift:676-711). */
int levo_q4_0_matvec_f64(const uint8_t *w, size_t w_bytes, int64_t out_dim,
                         int64_t in_dim, const float *x, size_t x_count, double *y);
/* MoESIMDOracle.q4MatvecFP64 (Sources/LeviathanCore/MoESIMDLowering.swift:934-977):
 * double input vector, bounded byte extent. */
int levo_q4_0_matvec_f64_xd(const uint8_t *w, size_t w_bytes, size_t byte_offset,
                            int64_t out_dim, int64_t in_dim, const double *x,
                            size_t x_count, double *y);

/* ---- Q6_K (Sources/LeviathanCore/Q6.swift:4-145,
 *           rust/crates/lev-cpu/src/lib.rs:197-294) ---- */
int levo_q6_k_decode_block(const uint8_t *block, float *out256);   /* Swift decodeBlock */
void levo_q6k_unpack(const uint8_t *block, int8_t *q256);          /* Rust q6k_unpack */
void levo_q6_k_dequant_block_f32(const uint8_t *block, float *out256);  /* Rust */
void levo_q6_k_dequant_block_f64(const uint8_t *block, double *out256); /* Rust */
int levo_q6_k_dequant(const uint8_t *w, size_t nblocks, float *out);
/* Swift Q6_K.matvecReference: f64 accumulate, rounded to f32 at the end. */
int levo_q6_k_matvec_ref(const uint8_t *w, size_t w_bytes, int64_t out_dim,
                         int64_t in_dim, const float *x, size_t x_count, float *y);
int levo_q6_k_matvec_ref_mt(const uint8_t *w, size_t w_bytes, int64_t out_dim,
                            int64_t in_dim, const float *x, size_t x_count, float *y,
                            int threads);
/* Swift Q6_K.matvecReferenceF64 == Rust matvec_q6k_f64. */
int levo_q6_k_matvec_f64(const uint8_t *w, size_t w_bytes, int64_t out_dim,
                         int64_t in_dim, const float *x, size_t x_count, double *y);
/* Rust matvec_q6k_f32: pure f32, ascending. */
int levo_q6_k_matvec_f32(const uint8_t *w, size_t w_bytes, int64_t out_dim,
                         int64_t in_dim, const float *x, size_t x_count, float *y);
/* ... with the rows split over `threads` threads (Model::matvec, lev-model lib.rs:184-199). */
int levo_q6_k_matvec_f32_mt(const uint8_t *w, size_t w_bytes, int64_t out_dim,
                            int64_t in_dim, const float *x, size_t x_count, float *y,
                            int threads);

/* ---- Q4_K (rust/crates/lev-cpu/src/lib.rs:62-195, test packer :380-394) ---- */
void levo_q4_k_unpack_scale_min(int j, const uint8_t *scales12, uint8_t *sc, uint8_t *mn);
void levo_q4_k_pack_scale_min(const uint8_t *sc8, const uint8_t *mn8, uint8_t *out12);
void levo_q4_k_dequant_block_f32(const uint8_t *block, float *out256);
void levo_q4_k_dequant_block_f64(const uint8_t *block, double *out256);
int levo_q4_k_dequant(const uint8_t *w, size_t nblocks, float *out);
int levo_q4_k_matvec_f32(const uint8_t *w, size_t w_bytes, int64_t rows, int64_t cols,
                         const float *x, size_t x_count, float *y);
int levo_q4_k_matvec_f32_mt(const uint8_t *w, size_t w_bytes, int64_t rows, int64_t cols,
                            const float *x, size_t x_count, float *y, int threads);
int levo_q4_k_matvec_f64(const uint8_t *w, size_t w_bytes, int64_t rows, int64_t cols,
                         const float *x, size_t x_count, double *y);

/* ---- int8 activations (rust/crates/lev-cpu/src/lib.rs:295-337) ---- */
int levo_quantize_q8(const float *x, size_t n, int8_t *q, float *d, float *s);

/* ---- RMSNorm ---- */
/* rust/crates/lev-model/src/lib.rs:110-114: f64 mean, (x*inv) as f32 * w. */
void levo_rmsnorm(const float *x, const float *w, float eps, size_t n, float *y);
/* g4_rmsnorm, Sources/LeviathanCore/Gemma4.swift:4247-4268: f32 serial;
 * w may be NULL (scale-free). */
void levo_rmsnorm_f32_serial(const float *x, const float *w, float eps, size_t n, float *y);
/* FP64 statement (Sources/LeviathanCore/RMSLowering.swift:350-386). */
void levo_rmsnorm_f64(const float *x, const float *w, double eps, size_t n, double *y);

/* ---- GELU-tanh * up ---- */
/* g4_tanh / g4_gelu_up_value, Sources/LeviathanCore/Gemma4.swift:4360-4377. */
float levo_stable_tanh_f32(float x);
float levo_gelu_up_f32(float g, float u);
/* MoESIMDOracle.geluTanhUp, Sources/LeviathanCore/MoESIMDLowering.swift:981-984. */
double levo_gelu_up_f64(double g, double u);

/* ---- argmax + margin (rust/crates/lev-model/src/lib.rs:395-416,
 *                        rust/crates/lev-forge/src/ops.rs:479-516) ---- */
size_t levo_argmax(const float *logits, size_t n);
float levo_top_margin(const float *logits, size_t n);

/* ---- normalised error (rust/crates/lev-cpu/src/lib.rs:341-353,
 *      Sources/LeviathanCore/MoESIMDLowering.swift:1034-1043) ----
 * Returns +inf where the Rust function returns None. */
double levo_max_rel_err(const float *got, size_t n_got, const double *ref, size_t n_ref);

/* ---- router (Sources/LeviathanCore/Gemma4.swift:3795-3810, kernel :4160-4171) ---- */
void levo_f32_matvec(const float *w, int64_t out_dim, int64_t in_dim, const float *x, float *y);
void levo_f32_matvec_f64(const float *w, int64_t out_dim, int64_t in_dim, const float *x, double *y);
/* scores[E] -> ids[K], weights[K]; expert_scale may be NULL (== 1). */
int levo_router_topk(const float *scores, int experts, int top_k,
                     const float *expert_scale, int32_t *ids, float *weights);

/* ---- MoE expert composite ----
 * The reference's serial per-slot loop (Sources/LeviathanCore/Gemma4.swift:3856-3880):
 * Q4_0 gate and up matvecs (kernel summation order), g4_gelu_up, Q4_0 down
 * matvec, axpy merge in slot order, all f32.  gate/up/down point at the
 * expert pools; expert e's slice starts at e*stride. */
int levo_moe_experts_f32(const uint8_t *gate, const uint8_t *up, const uint8_t *down,
                         size_t gate_stride, size_t up_stride, size_t down_stride,
                         int hidden, int inter, int top_k,
                         const int32_t *ids, const float *weights,
                         const float *x, float *y,
                         float *act_out /* [top_k][inter] or NULL */);
/* MoESIMDOracle.reference (Sources/LeviathanCore/MoESIMDLowering.swift:986-1030)
 * for the routed slots, plus the merged output in f64. */
int levo_moe_experts_f64(const uint8_t *gate, const uint8_t *up, const uint8_t *down,
                         size_t gate_stride, size_t up_stride, size_t down_stride,
                         int hidden, int inter, int top_k,
                         const int32_t *ids, const float *weights,
                         const float *x, double *y,
                         double *gate_out, double *up_out, double *act_out, double *dn_out);

/* ---- prefill GEMM oracle (rust/crates/lev-cli/src/main.rs:1201-1217,1266-1278) ----
 * W (Q4_K) dequantised in f32 then rounded to f16, X already f16 bits; f64
 * accumulate.  Computes rows row0, row0+row_step, ... for every token.
 * y_out is [tokens][n_sampled_rows]. */
int levo_q4_k_gemm_f16_oracle(const uint8_t *w, size_t w_bytes, int64_t rows, int64_t cols,
                              const uint16_t *x_f16, int64_t tokens,
                              int64_t row0, int64_t row_step, double *y_out);

/* Q6_K weights through the same gate (lev-forge/src/coopmat.rs:333-425). */
int levo_q6_k_gemm_f16_oracle(const uint8_t *w, size_t w_bytes, int64_t rows, int64_t cols,
                              const uint16_t *x_f16, int64_t tokens,
                              int64_t row0, int64_t row_step, double *y_out);

/* ---- synthetic inputs for the benchmark configurations ----
 * These are this build's own seeded generators (the reference only fixes
 * the distributions).  Normal draws use Box-Muller over SplitMix64. */
void levo_fill_normal(uint64_t seed, float mean, float sigma, float *out, size_t n);
void levo_synth_q4_0(uint64_t seed, float sigma_d, uint8_t *out, size_t nblocks);
void levo_synth_q6_k(uint64_t seed, float sigma_d, uint8_t *out, size_t nblocks);
void levo_synth_q4_k(uint64_t seed, float sigma_d, uint8_t *out, size_t nblocks);

#ifdef __cplusplus
}
#endif
#endif

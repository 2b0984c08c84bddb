/*
 * lev_oracle.c -- CPU restatement of Leviathan's quantized-matmul hot path.
 *
 * TEST INFRASTRUCTURE ONLY: see lev_oracle.h.  Build with
 *   gcc -O2 -ffp-contract=off -fPIC -shared -pthread lev_oracle.c -lm
 * (no -ffast-math; contraction off so f32 sums keep the source order).
 */
#include "lev_oracle.h"

#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ */
/* half precision: rust/crates/lev-cpu/src/lib.rs:14-60                */
/* ------------------------------------------------------------------ */

double levo_f16_to_f64(uint16_t h) {
    double sign = (h & 0x8000) ? -1.0 : 1.0;
    int exp = (h >> 10) & 0x1f;
    double mant = (double)(h & 0x3ff);
    if (exp == 0) return sign * mant * ldexp(1.0, -24);
    if (exp == 31) return mant == 0.0 ? sign * INFINITY : NAN;
    return sign * (1.0 + mant / 1024.0) * ldexp(1.0, exp - 15);
}

float levo_f16_to_f32(uint16_t h) { return (float)levo_f16_to_f64(h); }

uint16_t levo_f32_to_f16_bits(float v) {
    uint32_t b;
    memcpy(&b, &v, 4);
    uint16_t sign = (uint16_t)((b >> 16) & 0x8000);
    int exp = (int)((b >> 23) & 0xff);
    uint32_t mant = b & 0x7fffff;
    if (exp == 0xff) return (uint16_t)(sign | 0x7c00 | (mant != 0 ? 0x200 : 0));
    int e = exp - 127 + 15;
    if (e >= 31) return (uint16_t)(sign | 0x7c00);
    if (e <= 0) {
        if (e < -10) return sign;
        uint32_t m = mant | 0x800000;
        uint32_t shift = (uint32_t)(14 - e);
        uint16_t half = (uint16_t)(m >> shift);
        uint32_t rem = m & ((1u << shift) - 1u);
        uint32_t mid = 1u << (shift - 1);
        uint16_t round = (rem > mid || (rem == mid && (half & 1) == 1)) ? 1 : 0;
        return (uint16_t)(sign | (uint16_t)(half + round));
    }
    uint32_t half = ((uint32_t)e << 10) | (mant >> 13);
    uint32_t rem = mant & 0x1fff;
    uint32_t round = (rem > 0x1000 || (rem == 0x1000 && (half & 1) == 1)) ? 1 : 0;
    return (uint16_t)(sign | (uint16_t)(half + round));
}

/* ------------------------------------------------------------------ */
/* SplitMix64: RNG.swift:4-24, lev-cpu lib.rs:357-373                  */
/* ------------------------------------------------------------------ */

uint64_t levo_splitmix64_next(uint64_t *state) {
    *state += 0x9E3779B97F4A7C15ULL;
    uint64_t z = *state;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
    return z ^ (z >> 31);
}

float levo_next_uniform(uint64_t *state) {
    uint64_t u = levo_splitmix64_next(state) >> 11;
    return (float)((double)u / 9007199254740992.0) * 2.0f - 1.0f;
}

float levo_next_signed_unit(uint64_t *state) {
    float u = (float)(levo_splitmix64_next(state) >> 40) / (float)(1ULL << 24);
    return u * 2.0f - 1.0f;
}

void levo_fill_uniform(uint64_t seed, float *out, size_t n) {
    uint64_t s = seed;
    for (size_t i = 0; i < n; i++) out[i] = levo_next_uniform(&s);
}

void levo_fill_signed_unit(uint64_t seed, float *out, size_t n) {
    uint64_t s = seed;
    for (size_t i = 0; i < n; i++) out[i] = levo_next_signed_unit(&s);
}

/* ------------------------------------------------------------------ */
/* shared geometry checks                                              */
/* ------------------------------------------------------------------ */

#define LEVO_MAX_DIM ((int64_t)1 << 22)          /* ModelWorkloadLimits, Q4.swift:8-15 */
#define LEVO_MAX_WEIGHT_BYTES ((int64_t)32 << 30)

static int mul_overflow_i64(int64_t a, int64_t b, int64_t *out) {
    return __builtin_mul_overflow(a, b, out);
}

/* Q4.swift:87-101 / Q6.swift:67-80: dims, then byte count, then x count. */
static int check_geometry(int64_t out_dim, int64_t in_dim, int64_t block_values,
                          int64_t block_bytes, size_t w_bytes, size_t x_count,
                          int64_t *blocks_per_row) {
    if (in_dim <= 0 || out_dim <= 0 || in_dim % block_values != 0 ||
        in_dim > LEVO_MAX_DIM || out_dim > LEVO_MAX_DIM)
        return LEVO_BAD_DIMENSIONS;
    int64_t bpr = in_dim / block_values;
    int64_t need;
    if (mul_overflow_i64(out_dim, bpr * block_bytes, &need) || need > LEVO_MAX_WEIGHT_BYTES ||
        (int64_t)w_bytes != need)
        return LEVO_BAD_DIMENSIONS;
    if ((int64_t)x_count != in_dim) return LEVO_WRONG_INPUT_COUNT;
    *blocks_per_row = bpr;
    return LEVO_OK;
}

/* ------------------------------------------------------------------ */
/* Q4_0: Sources/LeviathanCore/Q4.swift:33-113                         */
/* ------------------------------------------------------------------ */

/* blockScale, Q4.swift:43-50 */
static int q4_0_block_scale(const uint8_t *block, float *d) {
    uint16_t bits = (uint16_t)(block[0] | (block[1] << 8));
    if ((bits & 0x7C00) == 0x7C00) return LEVO_NON_FINITE_SCALE;
    *d = levo_f16_to_f32(bits);
    return LEVO_OK;
}

/* decodeBlock, Q4.swift:54-69 */
int levo_q4_0_decode_block(const uint8_t *block, float *out) {
    float d;
    int st = q4_0_block_scale(block, &d);
    if (st) return st;
    for (int l = 0; l < 16; l++) {
        uint8_t byte = block[2 + l];
        out[l] = d * ((float)(byte & 0xF) - 8.0f);
        out[16 + l] = d * ((float)(byte >> 4) - 8.0f);
    }
    return LEVO_OK;
}

int levo_q4_0_dequant(const uint8_t *w, size_t nblocks, float *out) {
    for (size_t b = 0; b < nblocks; b++) {
        int st = levo_q4_0_decode_block(w + b * 18, out + b * 32);
        if (st) return st;
    }
    return LEVO_OK;
}

/* blockDot + row loop of matvecReference, Q4.swift:73-113 */
static int q4_0_rows_ref(const uint8_t *w, int64_t bpr, const float *x, float *y,
                         int64_t row0, int64_t row1) {
    float values[32];
    for (int64_t row = row0; row < row1; row++) {
        float sum = 0.0f;
        for (int64_t b = 0; b < bpr; b++) {
            const uint8_t *blk = w + (row * bpr + b) * 18;
            int st = levo_q4_0_decode_block(blk, values);
            if (st) return st;
            float part = 0.0f;
            for (int j = 0; j < 32; j++) {
                float xi = x[b * 32 + j];
                if (!isfinite(xi)) return LEVO_NON_FINITE_INPUT;
                part += values[j] * xi;
            }
            sum += part;
        }
        if (!isfinite(sum)) return LEVO_NON_FINITE_OUTPUT;
        y[row] = sum;
    }
    return LEVO_OK;
}

int levo_q4_0_matvec_ref(const uint8_t *w, size_t w_bytes, int64_t out_dim, int64_t in_dim,
                         const float *x, size_t x_count, float *y) {
    int64_t bpr;
    int st = check_geometry(out_dim, in_dim, 32, 18, w_bytes, x_count, &bpr);
    if (st) return st;
    return q4_0_rows_ref(w, bpr, x, y, 0, out_dim);
}

/* generic row-parallel driver (lev-model lib.rs:184-199: rows split evenly
 * over the available threads, each thread runs the scalar kernel). */
typedef int (*rows_fn)(const uint8_t *, int64_t, const float *, float *, int64_t, int64_t);
struct mt_job {
    rows_fn fn;
    const uint8_t *w;
    int64_t bpr;
    const float *x;
    float *y;
    int64_t row0, row1;
    int status;
};

static void *mt_entry(void *arg) {
    struct mt_job *j = (struct mt_job *)arg;
    j->status = j->fn(j->w, j->bpr, j->x, j->y, j->row0, j->row1);
    return NULL;
}

static int run_rows_mt(rows_fn fn, const uint8_t *w, int64_t bpr, const float *x, float *y,
                       int64_t rows, int threads) {
    if (threads < 1) threads = 1;
    if (threads > 256) threads = 256;
    if ((int64_t)threads > rows) threads = (int)rows;
    pthread_t tid[256];
    struct mt_job job[256];
    int64_t per = (rows + threads - 1) / threads;
    int n = 0;
    for (int t = 0; t < threads; t++) {
        int64_t r0 = (int64_t)t * per, r1 = r0 + per;
        if (r0 >= rows) break;
        if (r1 > rows) r1 = rows;
        job[n] = (struct mt_job){fn, w, bpr, x, y, r0, r1, 0};
        if (pthread_create(&tid[n], NULL, mt_entry, &job[n]) != 0) {
            job[n].status = fn(w, bpr, x, y, r0, r1);
            tid[n] = 0;
        }
        n++;
    }
    int st = LEVO_OK;
    for (int t = 0; t < n; t++) {
        if (tid[t]) pthread_join(tid[t], NULL);
        if (job[t].status && !st) st = job[t].status;
    }
    return st;
}

int levo_q4_0_matvec_ref_mt(const uint8_t *w, size_t w_bytes, int64_t out_dim, int64_t in_dim,
                            const float *x, size_t x_count, float *y, int threads) {
    int64_t bpr;
    int st = check_geometry(out_dim, in_dim, 32, 18, w_bytes, x_count, &bpr);
    if (st) return st;
    return run_rows_mt(q4_0_rows_ref, w, bpr, x, y, out_dim, threads);
}

/* leviathan_q4_matvec, Q4.swift:139-161: the serial kernel's order */
static void q4_0_rows_kernel_order(const uint8_t *w, int64_t bpr, const float *x, float *y,
                                   int64_t rows) {
    for (int64_t row = 0; row < rows; row++) {
        float sum = 0.0f;
        for (int64_t b = 0; b < bpr; b++) {
            const uint8_t *blk = w + (row * bpr + b) * 18;
            float d = levo_f16_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
            for (int l = 0; l < 16; l++) {
                uint8_t q = blk[2 + l];
                sum += d * ((float)(q & 0x0F) - 8.0f) * x[b * 32 + l];
                sum += d * ((float)(q >> 4) - 8.0f) * x[b * 32 + 16 + l];
            }
        }
        y[row] = sum;
    }
}

int levo_q4_0_matvec_kernel_order(const uint8_t *w, size_t w_bytes, int64_t out_dim,
                                  int64_t in_dim, const float *x, size_t x_count, float *y) {
    int64_t bpr;
    int st = check_geometry(out_dim, in_dim, 32, 18, w_bytes, x_count, &bpr);
    if (st) return st;
    for (int64_t i = 0; i < in_dim; i++)
        if (!isfinite(x[i])) return LEVO_NON_FINITE_INPUT;
    q4_0_rows_kernel_order(w, bpr, x, y, out_dim);
    for (int64_t r = 0; r < out_dim; r++)
        if (!isfinite(y[r])) return LEVO_NON_FINITE_OUTPUT;
    return LEVO_OK;
}

/* MoESIMDOracle.q4MatvecFP64, MoESIMDLowering.swift:934-977 */
int levo_q4_0_matvec_f64_xd(const uint8_t *w, size_t w_bytes, size_t byte_offset,
                            int64_t out_dim, int64_t in_dim, const double *x, size_t x_count,
                            double *y) {
    if (out_dim <= 0 || in_dim <= 0 || in_dim % 32 != 0 || (int64_t)x_count != in_dim)
        return LEVO_BAD_DIMENSIONS;
    for (int64_t i = 0; i < in_dim; i++)
        if (!isfinite(x[i])) return LEVO_NON_FINITE_INPUT;
    int64_t bpr = in_dim / 32, row_bytes, need, end;
    if (mul_overflow_i64(bpr, 18, &row_bytes) || mul_overflow_i64(out_dim, row_bytes, &need) ||
        __builtin_add_overflow((int64_t)byte_offset, need, &end) || end > (int64_t)w_bytes)
        return LEVO_BAD_DIMENSIONS;
    for (int64_t row = 0; row < out_dim; row++) {
        const uint8_t *rb = w + byte_offset + row * row_bytes;
        double sum = 0.0;
        for (int64_t b = 0; b < bpr; b++) {
            const uint8_t *blk = rb + b * 18;
            uint16_t bits = (uint16_t)(blk[0] | (blk[1] << 8));
            if ((bits & 0x7C00) == 0x7C00) return LEVO_NON_FINITE_SCALE;
            double d = levo_f16_to_f64(bits);
            for (int l = 0; l < 16; l++) {
                uint8_t q = blk[2 + l];
                sum += d * (double)((int)(q & 0x0F) - 8) * x[b * 32 + l];
                sum += d * (double)((int)(q >> 4) - 8) * x[b * 32 + 16 + l];
            }
        }
        if (!isfinite(sum)) return LEVO_NON_FINITE_OUTPUT;
        y[row] = sum;
    }
    return LEVO_OK;
}

/* Q4Oracle.matvecFP64, Q4Lowering.swift:676-711 */
int levo_q4_0_matvec_f64(const uint8_t *w, size_t w_bytes, int64_t out_dim, int64_t in_dim,
                         const float *x, size_t x_count, double *y) {
    if (in_dim <= 0 || out_dim <= 0 || in_dim % 32 != 0) return LEVO_BAD_DIMENSIONS;
    int64_t bpr = in_dim / 32;
    if ((int64_t)w_bytes != out_dim * bpr * 18 || (int64_t)x_count != in_dim)
        return LEVO_BAD_DIMENSIONS;
    for (int64_t i = 0; i < in_dim; i++)
        if (!isfinite(x[i])) return LEVO_NON_FINITE_INPUT;
    for (int64_t row = 0; row < out_dim; row++) {
        double sum = 0.0;
        for (int64_t b = 0; b < bpr; b++) {
            const uint8_t *blk = w + (row * bpr + b) * 18;
            uint16_t bits = (uint16_t)(blk[0] | (blk[1] << 8));
            if ((bits & 0x7C00) == 0x7C00) return LEVO_NON_FINITE_SCALE;
            double d = levo_f16_to_f64(bits);
            for (int l = 0; l < 16; l++) {
                uint8_t q = blk[2 + l];
                sum += d * ((double)(q & 0xF) - 8.0) * (double)x[b * 32 + l];
                sum += d * ((double)(q >> 4) - 8.0) * (double)x[b * 32 + 16 + l];
            }
        }
        if (!isfinite(sum)) return LEVO_NON_FINITE_OUTPUT;
        y[row] = sum;
    }
    return LEVO_OK;
}

/* ------------------------------------------------------------------ */
/* Q6_K: Sources/LeviathanCore/Q6.swift:4-145, lev-cpu lib.rs:197-294  */
/* ------------------------------------------------------------------ */

/* Swift Q6_K.decodeBlock, Q6.swift:23-62 */
int levo_q6_k_decode_block(const uint8_t *u8, float *out) {
    uint16_t dbits = (uint16_t)(u8[208] | (u8[209] << 8));
    if ((dbits & 0x7C00) == 0x7C00) return LEVO_NON_FINITE_SCALE;
    float d = levo_f16_to_f32(dbits);
    int scales[16];
    for (int i = 0; i < 16; i++) scales[i] = (int)(int8_t)u8[192 + i];
    for (int c = 0; c < 2; c++) {
        int ql = c * 64, qh = 128 + c * 32, sc = c * 8, base = c * 128;
        for (int l = 0; l < 32; l++) {
            int isub = l / 16;
            uint8_t b = u8[qh + l];
#define LEVEL(low, shift) (((low) | ((int)((b >> (shift)) & 3) << 4)) - 32)
            out[base + l] = d * (float)scales[sc + isub + 0] * (float)LEVEL((int)(u8[ql + l] & 0xF), 0);
            out[base + 32 + l] =
                d * (float)scales[sc + isub + 2] * (float)LEVEL((int)(u8[ql + 32 + l] & 0xF), 2);
            out[base + 64 + l] = d * (float)scales[sc + isub + 4] * (float)LEVEL((int)(u8[ql + l] >> 4), 4);
            out[base + 96 + l] =
                d * (float)scales[sc + isub + 6] * (float)LEVEL((int)(u8[ql + 32 + l] >> 4), 6);
#undef LEVEL
        }
    }
    return LEVO_OK;
}

/* Rust q6k_unpack, lev-cpu lib.rs:203-216 */
void levo_q6k_unpack(const uint8_t *block, int8_t *q) {
    const uint8_t *ql0 = block, *qh0 = block + 128;
    for (int half = 0; half < 2; half++) {
        const uint8_t *ql = ql0 + half * 64, *qh = qh0 + half * 32;
        for (int l = 0; l < 32; l++) {
            uint8_t h = qh[l];
            q[half * 128 + l] = (int8_t)((int8_t)((ql[l] & 0x0F) | ((h & 3) << 4)) - 32);
            q[half * 128 + l + 32] = (int8_t)((int8_t)((ql[l + 32] & 0x0F) | (((h >> 2) & 3) << 4)) - 32);
            q[half * 128 + l + 64] = (int8_t)((int8_t)((ql[l] >> 4) | (((h >> 4) & 3) << 4)) - 32);
            q[half * 128 + l + 96] = (int8_t)((int8_t)((ql[l + 32] >> 4) | (((h >> 6) & 3) << 4)) - 32);
        }
    }
}

/* Rust dequant_q6k_block_f32 / _f64, lev-cpu lib.rs:218-244 */
void levo_q6_k_dequant_block_f32(const uint8_t *block, float *out) {
    int8_t q[256];
    levo_q6k_unpack(block, q);
    float d = (float)levo_f16_to_f64((uint16_t)(block[208] | (block[209] << 8)));
    for (int e = 0; e < 256; e++) out[e] = d * (float)(int8_t)block[192 + e / 16] * (float)q[e];
}

void levo_q6_k_dequant_block_f64(const uint8_t *block, double *out) {
    int8_t q[256];
    levo_q6k_unpack(block, q);
    double d = levo_f16_to_f64((uint16_t)(block[208] | (block[209] << 8)));
    for (int e = 0; e < 256; e++) out[e] = d * (double)(int8_t)block[192 + e / 16] * (double)q[e];
}

int levo_q6_k_dequant(const uint8_t *w, size_t nblocks, float *out) {
    for (size_t b = 0; b < nblocks; b++) {
        int st = levo_q6_k_decode_block(w + b * 210, out + b * 256);
        if (st) return st;
    }
    return LEVO_OK;
}

/* Swift Q6_K.matvecReference rows, Q6.swift:89-108 */
static int q6_k_rows_ref(const uint8_t *w, int64_t bpr, const float *x, float *y, int64_t row0,
                         int64_t row1) {
    float values[256];
    for (int64_t row = row0; row < row1; row++) {
        double sum = 0.0;
        for (int64_t b = 0; b < bpr; b++) {
            int st = levo_q6_k_decode_block(w + (row * bpr + b) * 210, values);
            if (st) return st;
            for (int j = 0; j < 256; j++) {
                float xi = x[b * 256 + j];
                if (!isfinite(xi)) return LEVO_NON_FINITE_INPUT;
                sum += (double)values[j] * (double)xi;
            }
        }
        float f = (float)sum;
        if (!isfinite(f)) return LEVO_NON_FINITE_OUTPUT;
        y[row] = f;
    }
    return LEVO_OK;
}

int levo_q6_k_matvec_ref(const uint8_t *w, size_t w_bytes, int64_t out_dim, int64_t in_dim,
                         const float *x, size_t x_count, float *y) {
    int64_t bpr;
    int st = check_geometry(out_dim, in_dim, 256, 210, w_bytes, x_count, &bpr);
    if (st) return st;
    return q6_k_rows_ref(w, bpr, x, y, 0, out_dim);
}

int levo_q6_k_matvec_ref_mt(const uint8_t *w, size_t w_bytes, int64_t out_dim, int64_t in_dim,
                            const float *x, size_t x_count, float *y, int threads) {
    int64_t bpr;
    int st = check_geometry(out_dim, in_dim, 256, 210, w_bytes, x_count, &bpr);
    if (st) return st;
    return run_rows_mt(q6_k_rows_ref, w, bpr, x, y, out_dim, threads);
}

/* Swift Q6_K.matvecReferenceF64, Q6.swift:112-145 */
int levo_q6_k_matvec_f64(const uint8_t *w, size_t w_bytes, int64_t out_dim, int64_t in_dim,
                         const float *x, size_t x_count, double *y) {
    int64_t bpr;
    int st = check_geometry(out_dim, in_dim, 256, 210, w_bytes, x_count, &bpr);
    if (st) return st;
    for (int64_t i = 0; i < in_dim; i++)
        if (!isfinite(x[i])) return LEVO_NON_FINITE_INPUT;
    float values[256];
    for (int64_t row = 0; row < out_dim; row++) {
        double sum = 0.0;
        for (int64_t b = 0; b < bpr; b++) {
            st = levo_q6_k_decode_block(w + (row * bpr + b) * 210, values);
            if (st) return st;
            for (int j = 0; j < 256; j++) sum += (double)values[j] * (double)x[b * 256 + j];
        }
        if (!isfinite(sum)) return LEVO_NON_FINITE_OUTPUT;
        y[row] = sum;
    }
    return LEVO_OK;
}

/* Rust matvec_q6k_f32, lev-cpu lib.rs:261-276 (shape errors :246-259) */
static int q6_k_rows_f32(const uint8_t *w, int64_t bpr, const float *x, float *y, int64_t row0, int64_t row1) {
    const int64_t row_bytes = bpr * 210;
    float tmp[256];
    for (int64_t r = row0; r < row1; r++) {
        float sum = 0.0f;
        for (int64_t b = 0; b < bpr; b++) {
            levo_q6_k_dequant_block_f32(w + r * row_bytes + b * 210, tmp);
            for (int i = 0; i < 256; i++) sum += tmp[i] * x[b * 256 + i];
        }
        y[r] = sum;
    }
    return LEVO_OK;
}

static int q6_k_check_shape_f32(size_t w_bytes, int64_t rows, int64_t cols, size_t x_count) {
    if (cols == 0 || cols % 256 != 0 || rows < 0) return LEVO_BAD_DIMENSIONS;
    int64_t row_bytes = cols / 256 * 210, expected;
    if (mul_overflow_i64(rows, row_bytes, &expected) || (int64_t)w_bytes != expected)
        return LEVO_BAD_DIMENSIONS;
    if ((int64_t)x_count != cols) return LEVO_WRONG_INPUT_COUNT;
    return LEVO_OK;
}

int levo_q6_k_matvec_f32(const uint8_t *w, size_t w_bytes, int64_t rows, int64_t cols,
                         const float *x, size_t x_count, float *y) {
    int st = q6_k_check_shape_f32(w_bytes, rows, cols, x_count);
    if (st) return st;
    return q6_k_rows_f32(w, cols / 256, x, y, 0, rows);
}

/* the same rows split over threads, as Model::matvec does (lev-model lib.rs:184-199) */
int levo_q6_k_matvec_f32_mt(const uint8_t *w, size_t w_bytes, int64_t rows, int64_t cols,
                            const float *x, size_t x_count, float *y, int threads) {
    int st = q6_k_check_shape_f32(w_bytes, rows, cols, x_count);
    if (st) return st;
    if (rows == 0) return LEVO_OK;
    return run_rows_mt(q6_k_rows_f32, w, cols / 256, x, y, rows, threads);
}

/* ------------------------------------------------------------------ */
/* Q4_K: rust/crates/lev-cpu/src/lib.rs:62-195                         */
/* ------------------------------------------------------------------ */

/* unpack_scale_min, lib.rs:64-74 */
void levo_q4_k_unpack_scale_min(int j, const uint8_t *scales, uint8_t *sc, uint8_t *mn) {
    if (j < 4) {
        *sc = scales[j] & 63;
        *mn = scales[j + 4] & 63;
    } else {
        *sc = (uint8_t)((scales[j + 4] & 0x0F) | ((scales[j - 4] >> 6) << 4));
        *mn = (uint8_t)((scales[j + 4] >> 4) | ((scales[j] >> 6) << 4));
    }
}

/* the ggml encoder's packing, restated from the reference test, lib.rs:380-394 */
void levo_q4_k_pack_scale_min(const uint8_t *sc, const uint8_t *mn, uint8_t *s) {
    memset(s, 0, 12);
    for (int j = 0; j < 8; j++) {
        uint8_t ls = sc[j], lm = mn[j];
        if (j < 4) {
            s[j] = ls;
            s[j + 4] = lm;
        } else {
            s[j + 4] = (uint8_t)((ls & 0x0F) | ((lm & 0x0F) << 4));
            s[j - 4] |= (uint8_t)((ls >> 4) << 6);
            s[j] |= (uint8_t)((lm >> 4) << 6);
        }
    }
}

/* dequant_block_f32, lib.rs:111-131 */
void levo_q4_k_dequant_block_f32(const uint8_t *block, float *out) {
    float d = levo_f16_to_f32((uint16_t)(block[0] | (block[1] << 8)));
    float dmin = levo_f16_to_f32((uint16_t)(block[2] | (block[3] << 8)));
    const uint8_t *scales = block + 4, *qs = block + 16;
    int is = 0;
    for (int chunk = 0; chunk < 4; chunk++) {
        const uint8_t *q = qs + chunk * 32;
        uint8_t sc1, m1, sc2, m2;
        levo_q4_k_unpack_scale_min(is, scales, &sc1, &m1);
        levo_q4_k_unpack_scale_min(is + 1, scales, &sc2, &m2);
        float d1 = d * (float)sc1, mm1 = dmin * (float)m1;
        float d2 = d * (float)sc2, mm2 = dmin * (float)m2;
        int o = chunk * 64;
        for (int l = 0; l < 32; l++) {
            out[o + l] = d1 * (float)(q[l] & 0x0F) - mm1;
            out[o + 32 + l] = d2 * (float)(q[l] >> 4) - mm2;
        }
        is += 2;
    }
}

/* dequant_block_f64, lib.rs:134-154 */
void levo_q4_k_dequant_block_f64(const uint8_t *block, double *out) {
    double d = levo_f16_to_f64((uint16_t)(block[0] | (block[1] << 8)));
    double dmin = levo_f16_to_f64((uint16_t)(block[2] | (block[3] << 8)));
    const uint8_t *scales = block + 4, *qs = block + 16;
    int is = 0;
    for (int chunk = 0; chunk < 4; chunk++) {
        const uint8_t *q = qs + chunk * 32;
        uint8_t sc1, m1, sc2, m2;
        levo_q4_k_unpack_scale_min(is, scales, &sc1, &m1);
        levo_q4_k_unpack_scale_min(is + 1, scales, &sc2, &m2);
        double d1 = d * (double)sc1, mm1 = dmin * (double)m1;
        double d2 = d * (double)sc2, mm2 = dmin * (double)m2;
        int o = chunk * 64;
        for (int l = 0; l < 32; l++) {
            out[o + l] = d1 * (double)(q[l] & 0x0F) - mm1;
            out[o + 32 + l] = d2 * (double)(q[l] >> 4) - mm2;
        }
        is += 2;
    }
}

int levo_q4_k_dequant(const uint8_t *w, size_t nblocks, float *out) {
    for (size_t b = 0; b < nblocks; b++) levo_q4_k_dequant_block_f32(w + b * 144, out + b * 256);
    return LEVO_OK;
}

/* check_shape, lib.rs:94-108 */
static int q4_k_check_shape(size_t w_bytes, int64_t rows, int64_t cols, size_t x_count,
                            int64_t *row_bytes) {
    if (cols == 0 || cols % 256 != 0 || rows < 0) return LEVO_BAD_DIMENSIONS;
    *row_bytes = cols / 256 * 144;
    int64_t expected;
    if (mul_overflow_i64(rows, *row_bytes, &expected) || (int64_t)w_bytes != expected)
        return LEVO_BAD_DIMENSIONS;
    if ((int64_t)x_count != cols) return LEVO_WRONG_INPUT_COUNT;
    return LEVO_OK;
}

/* matvec_q4k_f32 rows, lib.rs:158-175 */
static int q4_k_rows_f32(const uint8_t *w, int64_t bpr, const float *x, float *y, int64_t row0,
                         int64_t row1) {
    float tmp[256];
    for (int64_t r = row0; r < row1; r++) {
        float sum = 0.0f;
        for (int64_t b = 0; b < bpr; b++) {
            levo_q4_k_dequant_block_f32(w + (r * bpr + b) * 144, tmp);
            const float *xs = x + b * 256;
            for (int i = 0; i < 256; i++) sum += tmp[i] * xs[i];
        }
        y[r] = sum;
    }
    return LEVO_OK;
}

int levo_q4_k_matvec_f32(const uint8_t *w, size_t w_bytes, int64_t rows, int64_t cols,
                         const float *x, size_t x_count, float *y) {
    int64_t row_bytes;
    int st = q4_k_check_shape(w_bytes, rows, cols, x_count, &row_bytes);
    if (st) return st;
    return q4_k_rows_f32(w, cols / 256, x, y, 0, rows);
}

int levo_q4_k_matvec_f32_mt(const uint8_t *w, size_t w_bytes, int64_t rows, int64_t cols,
                            const float *x, size_t x_count, float *y, int threads) {
    int64_t row_bytes;
    int st = q4_k_check_shape(w_bytes, rows, cols, x_count, &row_bytes);
    if (st) return st;
    if (rows == 0) return LEVO_OK;
    return run_rows_mt(q4_k_rows_f32, w, cols / 256, x, y, rows, threads);
}

/* matvec_q4k_f64, lib.rs:178-195 */
int levo_q4_k_matvec_f64(const uint8_t *w, size_t w_bytes, int64_t rows, int64_t cols,
                         const float *x, size_t x_count, double *y) {
    int64_t row_bytes;
    int st = q4_k_check_shape(w_bytes, rows, cols, x_count, &row_bytes);
    if (st) return st;
    double tmp[256];
    for (int64_t r = 0; r < rows; r++) {
        double sum = 0.0;
        for (int64_t b = 0; b < cols / 256; b++) {
            levo_q4_k_dequant_block_f64(w + r * row_bytes + b * 144, tmp);
            const float *xs = x + b * 256;
            for (int i = 0; i < 256; i++) sum += tmp[i] * (double)xs[i];
        }
        y[r] = sum;
    }
    return LEVO_OK;
}

/* ------------------------------------------------------------------ */
/* int8 activations: lev-cpu lib.rs:295-322                            */
/* ------------------------------------------------------------------ */

int levo_quantize_q8(const float *x, size_t n, int8_t *q, float *d, float *s) {
    if (n % 32 != 0) return LEVO_BAD_DIMENSIONS;
    for (size_t g = 0; g < n / 32; g++) {
        const float *v = x + g * 32;
        float amax = 0.0f;
        for (int i = 0; i < 32; i++) amax = fmaxf(amax, fabsf(v[i]));
        float dd = 0.0f, id = 0.0f;
        if (amax > 0.0f) {
            dd = amax / 127.0f;
            id = 127.0f / amax;
        }
        int sum = 0;
        for (int i = 0; i < 32; i++) {
            int qi = (int)rintf(v[i] * id); /* round half to even */
            sum += qi;
            q[g * 32 + i] = (int8_t)qi;
        }
        d[g] = dd;
        s[g] = dd * (float)sum;
    }
    return LEVO_OK;
}

/* ------------------------------------------------------------------ */
/* RMSNorm                                                             */
/* ------------------------------------------------------------------ */

/* lev-model lib.rs:110-114 */
void levo_rmsnorm(const float *x, const float *w, float eps, size_t n, float *y) {
    double ms = 0.0;
    for (size_t i = 0; i < n; i++) ms += (double)x[i] * (double)x[i];
    ms /= (double)n;
    double inv = 1.0 / sqrt(ms + (double)eps);
    for (size_t i = 0; i < n; i++) y[i] = (float)((double)x[i] * inv) * w[i];
}

/* g4_rmsnorm, Gemma4.swift:4247-4268 */
void levo_rmsnorm_f32_serial(const float *x, const float *w, float eps, size_t n, float *y) {
    float ms = 0.0f;
    for (size_t i = 0; i < n; i++) ms += x[i] * x[i];
    ms = ms / (float)n + eps;
    float inv = 1.0f / sqrtf(ms);
    for (size_t i = 0; i < n; i++) y[i] = x[i] * inv * (w ? w[i] : 1.0f);
}

/* RMSOracle.rmsnormFP64, RMSLowering.swift:350-386 */
void levo_rmsnorm_f64(const float *x, const float *w, double eps, size_t n, double *y) {
    double ms = 0.0;
    for (size_t i = 0; i < n; i++) {
        double d = (double)x[i];
        ms += d * d;
    }
    double inv = 1.0 / sqrt(ms / (double)n + eps);
    for (size_t i = 0; i < n; i++) y[i] = (double)x[i] * inv * (w ? (double)w[i] : 1.0);
}

/* ------------------------------------------------------------------ */
/* GELU-tanh * up                                                      */
/* ------------------------------------------------------------------ */

/* g4_tanh, Gemma4.swift:4364-4367 */
float levo_stable_tanh_f32(float x) {
    float e = expf(-2.0f * fabsf(x));
    return copysignf((1.0f - e) / (1.0f + e), x);
}

/* g4_gelu_up_value, Gemma4.swift:4373-4377 */
float levo_gelu_up_f32(float g, float u) {
    float inner = 0.7978845608028654f * (g + 0.044715f * g * g * g);
    float gelu = 0.5f * g * (1.0f + levo_stable_tanh_f32(inner));
    return gelu * u;
}

/* MoESIMDOracle.geluTanhUp, MoESIMDLowering.swift:981-984 */
double levo_gelu_up_f64(double g, double u) {
    double inner = 0.7978845608028654 * (g + 0.044715 * g * g * g);
    return 0.5 * g * (1.0 + tanh(inner)) * u;
}

/* ------------------------------------------------------------------ */
/* argmax + margin: lev-model lib.rs:395-416                           */
/* ------------------------------------------------------------------ */

size_t levo_argmax(const float *logits, size_t n) {
    size_t best = 0;
    for (size_t i = 0; i < n; i++)
        if (logits[i] > logits[best]) best = i;
    return best;
}

float levo_top_margin(const float *logits, size_t n) {
    float a = -INFINITY, b = -INFINITY;
    for (size_t i = 0; i < n; i++) {
        float v = logits[i];
        if (v > a) {
            b = a;
            a = v;
        } else if (v > b) {
            b = v;
        }
    }
    return a - b;
}

/* ------------------------------------------------------------------ */
/* error metric: lev-cpu lib.rs:341-353                                */
/* ------------------------------------------------------------------ */

double levo_max_rel_err(const float *got, size_t n_got, const double *ref, size_t n_ref) {
    if (n_got != n_ref || n_got == 0) return INFINITY;
    double worst = 0.0;
    for (size_t i = 0; i < n_got; i++) {
        if (!isfinite(got[i]) || !isfinite(ref[i])) return INFINITY;
        double e = fabs((double)got[i] - ref[i]) / fmax(fabs(ref[i]), 1.0);
        if (e > worst) worst = e;
    }
    return worst;
}

/* ------------------------------------------------------------------ */
/* router: Gemma4.swift:3795-3810, g4_f32_matvec :4160-4171            */
/* ------------------------------------------------------------------ */

void levo_f32_matvec(const float *w, int64_t out_dim, int64_t in_dim, const float *x, float *y) {
    for (int64_t r = 0; r < out_dim; r++) {
        float sum = 0.0f;
        for (int64_t i = 0; i < in_dim; i++) sum += w[r * in_dim + i] * x[i];
        y[r] = sum;
    }
}

void levo_f32_matvec_f64(const float *w, int64_t out_dim, int64_t in_dim, const float *x,
                         double *y) {
    for (int64_t r = 0; r < out_dim; r++) {
        double sum = 0.0;
        for (int64_t i = 0; i < in_dim; i++) sum += (double)w[r * in_dim + i] * (double)x[i];
        y[r] = sum;
    }
}

/* Gemma4.swift:3798-3810.  The comparator `p[a] > p[b] || (p[a] == p[b] && a < b)`
 * is a strict total order on distinct indices, so any correct sort gives the
 * same permutation; selection of the K first is done by repeated extraction. */
int levo_router_topk(const float *scores, int experts, int top_k, const float *expert_scale,
                     int32_t *ids, float *weights) {
    if (experts <= 0 || top_k <= 0 || top_k > experts) return LEVO_BAD_DIMENSIONS;
    for (int i = 0; i < experts; i++)
        if (!isfinite(scores[i])) return LEVO_NON_FINITE_INPUT;
    float max_score = scores[0];
    for (int i = 1; i < experts; i++)
        if (scores[i] > max_score) max_score = scores[i];
    double *probs = (double *)malloc(sizeof(double) * (size_t)experts);
    char *taken = (char *)calloc((size_t)experts, 1);
    if (!probs || !taken) {
        free(probs);
        free(taken);
        return LEVO_INVALID_ARGUMENT;
    }
    double sum_exp = 0.0;
    for (int i = 0; i < experts; i++) {
        probs[i] = exp((double)(scores[i] - max_score)); /* subtraction in f32 */
        sum_exp += probs[i];
    }
    for (int i = 0; i < experts; i++) probs[i] /= sum_exp;
    double prob_sum = 0.0;
    for (int k = 0; k < top_k; k++) {
        int best = -1;
        for (int i = 0; i < experts; i++) {
            if (taken[i]) continue;
            if (best < 0 || probs[i] > probs[best]) best = i; /* ties keep lower index */
        }
        taken[best] = 1;
        ids[k] = best;
        prob_sum += probs[best];
    }
    for (int k = 0; k < top_k; k++)
        weights[k] = (float)(probs[ids[k]] / prob_sum) * (expert_scale ? expert_scale[ids[k]] : 1.0f);
    free(probs);
    free(taken);
    return LEVO_OK;
}

/* ------------------------------------------------------------------ */
/* MoE expert composite                                                */
/* ------------------------------------------------------------------ */

/* Gemma4.swift:3856-3880 with the kernels it dispatches:
 * g4_q4_matvec (:3931), g4_gelu_up (:4380), g4_axpy (:4459). */
int levo_moe_experts_f32(const uint8_t *gate, const uint8_t *up, const uint8_t *down,
                         size_t gate_stride, size_t up_stride, size_t down_stride, int hidden,
                         int inter, int top_k, const int32_t *ids, const float *weights,
                         const float *x, float *y, float *act_out) {
    if (hidden <= 0 || inter <= 0 || top_k <= 0 || hidden % 32 != 0 || inter % 32 != 0)
        return LEVO_BAD_DIMENSIONS;
    for (int i = 0; i < hidden; i++)
        if (!isfinite(x[i])) return LEVO_NON_FINITE_INPUT;
    float *g = (float *)malloc(sizeof(float) * (size_t)inter * 3 + sizeof(float) * (size_t)hidden);
    if (!g) return LEVO_INVALID_ARGUMENT;
    float *u = g + inter, *act = u + inter, *t2 = act + inter;
    int64_t hb = hidden / 32, ib = inter / 32;
    memset(y, 0, sizeof(float) * (size_t)hidden); /* MoE accumulator */
    for (int slot = 0; slot < top_k; slot++) {
        int e = ids[slot];
        q4_0_rows_kernel_order(gate + (size_t)e * gate_stride, hb, x, g, inter);
        q4_0_rows_kernel_order(up + (size_t)e * up_stride, hb, x, u, inter);
        for (int i = 0; i < inter; i++) act[i] = levo_gelu_up_f32(g[i], u[i]);
        if (act_out) memcpy(act_out + (size_t)slot * inter, act, sizeof(float) * (size_t)inter);
        q4_0_rows_kernel_order(down + (size_t)e * down_stride, ib, act, t2, hidden);
        float c = weights[slot];
        for (int i = 0; i < hidden; i++) y[i] += c * t2[i];
    }
    free(g);
    return LEVO_OK;
}

/* MoESIMDOracle.reference, MoESIMDLowering.swift:986-1030 */
int levo_moe_experts_f64(const uint8_t *gate, const uint8_t *up, const uint8_t *down,
                         size_t gate_stride, size_t up_stride, size_t down_stride, int hidden,
                         int inter, int top_k, const int32_t *ids, const float *weights,
                         const float *x, double *y, double *gate_out, double *up_out,
                         double *act_out, double *dn_out) {
    if (hidden <= 0 || inter <= 0 || top_k <= 0 || hidden % 32 != 0 || inter % 32 != 0)
        return LEVO_BAD_DIMENSIONS;
    for (int i = 0; i < hidden; i++)
        if (!isfinite(x[i])) return LEVO_NON_FINITE_INPUT;
    size_t gu_bytes = (size_t)inter * (size_t)(hidden / 32) * 18;
    size_t dn_bytes = (size_t)hidden * (size_t)(inter / 32) * 18;
    double *xd = (double *)malloc(sizeof(double) * ((size_t)hidden * 2 + (size_t)inter * 3));
    if (!xd) return LEVO_INVALID_ARGUMENT;
    double *g = xd + hidden, *u = g + inter, *a = u + inter, *d = a + inter;
    for (int i = 0; i < hidden; i++) xd[i] = (double)x[i];
    if (y)
        for (int i = 0; i < hidden; i++) y[i] = 0.0;
    int st = LEVO_OK;
    for (int slot = 0; slot < top_k && !st; slot++) {
        int e = ids[slot];
        st = levo_q4_0_matvec_f64_xd(gate + (size_t)e * gate_stride, gu_bytes, 0, inter, hidden,
                                     xd, (size_t)hidden, g);
        if (st) break;
        st = levo_q4_0_matvec_f64_xd(up + (size_t)e * up_stride, gu_bytes, 0, inter, hidden, xd,
                                     (size_t)hidden, u);
        if (st) break;
        for (int i = 0; i < inter; i++) {
            a[i] = levo_gelu_up_f64(g[i], u[i]);
            if (!isfinite(a[i])) {
                st = LEVO_NON_FINITE_OUTPUT;
                break;
            }
        }
        if (st) break;
        st = levo_q4_0_matvec_f64_xd(down + (size_t)e * down_stride, dn_bytes, 0, hidden, inter,
                                     a, (size_t)inter, d);
        if (st) break;
        if (gate_out) memcpy(gate_out + (size_t)slot * inter, g, sizeof(double) * (size_t)inter);
        if (up_out) memcpy(up_out + (size_t)slot * inter, u, sizeof(double) * (size_t)inter);
        if (act_out) memcpy(act_out + (size_t)slot * inter, a, sizeof(double) * (size_t)inter);
        if (dn_out) memcpy(dn_out + (size_t)slot * hidden, d, sizeof(double) * (size_t)hidden);
        if (y)
            for (int i = 0; i < hidden; i++) y[i] += (double)weights[slot] * d[i];
    }
    free(xd);
    return st;
}

/* ------------------------------------------------------------------ */
/* prefill GEMM oracle: lev-cli main.rs:1201-1217, 1266-1278           */
/* ------------------------------------------------------------------ */

int levo_q4_k_gemm_f16_oracle(const uint8_t *w, size_t w_bytes, int64_t rows, int64_t cols,
                              const uint16_t *x_f16, int64_t tokens, int64_t row0,
                              int64_t row_step, double *y_out) {
    int64_t row_bytes;
    int st = q4_k_check_shape(w_bytes, rows, cols, (size_t)cols, &row_bytes);
    if (st) return st;
    if (tokens <= 0 || row_step <= 0 || row0 < 0) return LEVO_BAD_DIMENSIONS;
    int64_t n_rows = row0 < rows ? (rows - row0 + row_step - 1) / row_step : 0;
    double *wr = (double *)malloc(sizeof(double) * (size_t)cols);
    double *xr = (double *)malloc(sizeof(double) * (size_t)cols * (size_t)tokens);
    if (!wr || !xr) {
        free(wr);
        free(xr);
        return LEVO_INVALID_ARGUMENT;
    }
    for (int64_t i = 0; i < cols * tokens; i++) xr[i] = levo_f16_to_f64(x_f16[i]);
    float tmp[256];
    int64_t k = 0;
    for (int64_t r = row0; r < rows; r += row_step, k++) {
        for (int64_t b = 0; b < cols / 256; b++) {
            levo_q4_k_dequant_block_f32(w + r * row_bytes + b * 144, tmp);
            for (int i = 0; i < 256; i++)
                wr[b * 256 + i] = levo_f16_to_f64(levo_f32_to_f16_bits(tmp[i]));
        }
        for (int64_t t = 0; t < tokens; t++) {
            double acc = 0.0;
            const double *xt = xr + t * cols;
            for (int64_t c = 0; c < cols; c++) acc += wr[c] * xt[c];
            y_out[t * n_rows + k] = acc;
        }
    }
    free(wr);
    free(xr);
    return LEVO_OK;
}

/* The same gate for Q6_K weights (q6k gemm blocked, lev-forge coopmat.rs:333-425:
 * float16_t(ds * float(q - 32)) with ds = d * float(scale)): the f32 value of
 * decodeBlock, d * sc * level evaluated left to right, rounded to f16. */
int levo_q6_k_gemm_f16_oracle(const uint8_t *w, size_t w_bytes, int64_t rows, int64_t cols,
                              const uint16_t *x_f16, int64_t tokens, int64_t row0,
                              int64_t row_step, double *y_out) {
    if (rows <= 0 || cols <= 0 || cols % 256 != 0) return LEVO_BAD_DIMENSIONS;
    const int64_t row_bytes = cols / 256 * 210;
    if ((uint64_t)rows * (uint64_t)row_bytes > (uint64_t)w_bytes) return LEVO_BAD_DIMENSIONS;
    if (tokens <= 0 || row_step <= 0 || row0 < 0) return LEVO_BAD_DIMENSIONS;
    int64_t n_rows = row0 < rows ? (rows - row0 + row_step - 1) / row_step : 0;
    double *wr = (double *)malloc(sizeof(double) * (size_t)cols);
    double *xr = (double *)malloc(sizeof(double) * (size_t)cols * (size_t)tokens);
    if (!wr || !xr) {
        free(wr);
        free(xr);
        return LEVO_INVALID_ARGUMENT;
    }
    for (int64_t i = 0; i < cols * tokens; i++) xr[i] = levo_f16_to_f64(x_f16[i]);
    float tmp[256];
    int st = LEVO_OK;
    int64_t k = 0;
    for (int64_t r = row0; r < rows && st == LEVO_OK; r += row_step, k++) {
        for (int64_t b = 0; b < cols / 256; b++) {
            st = levo_q6_k_decode_block(w + r * row_bytes + b * 210, tmp);
            if (st) break;
            for (int i = 0; i < 256; i++)
                wr[b * 256 + i] = levo_f16_to_f64(levo_f32_to_f16_bits(tmp[i]));
        }
        if (st) break;
        for (int64_t t = 0; t < tokens; t++) {
            double acc = 0.0;
            const double *xt = xr + t * cols;
            for (int64_t c = 0; c < cols; c++) acc += wr[c] * xt[c];
            y_out[t * n_rows + k] = acc;
        }
    }
    free(wr);
    free(xr);
    return st;
}

/* ------------------------------------------------------------------ */
/* synthetic inputs (this build's own seeded generators)               */
/* ------------------------------------------------------------------ */

static double unit_open(uint64_t *s) { /* (0, 1] */
    return ((double)(levo_splitmix64_next(s) >> 11) + 1.0) / 9007199254740992.0;
}

static double next_normal(uint64_t *s) { /* Box-Muller, one draw per call */
    double u1 = unit_open(s), u2 = unit_open(s);
    return sqrt(-2.0 * log(u1)) * cos(6.283185307179586476925286766559 * u2);
}

void levo_fill_normal(uint64_t seed, float mean, float sigma, float *out, size_t n) {
    uint64_t s = seed;
    for (size_t i = 0; i < n; i++) out[i] = (float)((double)mean + (double)sigma * next_normal(&s));
}

static uint16_t abs_normal_f16(uint64_t *s, float sigma) {
    uint16_t h = levo_f32_to_f16_bits((float)fabs((double)sigma * next_normal(s)));
    if ((h & 0x7C00) == 0x7C00) h = 0x3C00; /* never Inf/NaN */
    return h;
}

static void fill_bytes(uint64_t *s, uint8_t *out, size_t n) {
    size_t i = 0;
    while (i < n) {
        uint64_t v = levo_splitmix64_next(s);
        for (int k = 0; k < 8 && i < n; k++, i++) out[i] = (uint8_t)(v >> (8 * k));
    }
}

/* Q4_0 block: fp16 d = |N(0, sigma_d)|, 16 uniformly random code bytes. */
void levo_synth_q4_0(uint64_t seed, float sigma_d, uint8_t *out, size_t nblocks) {
    uint64_t s = seed;
    for (size_t b = 0; b < nblocks; b++) {
        uint8_t *blk = out + b * 18;
        uint16_t h = abs_normal_f16(&s, sigma_d);
        blk[0] = (uint8_t)(h & 0xFF);
        blk[1] = (uint8_t)(h >> 8);
        fill_bytes(&s, blk + 2, 16);
    }
}

/* Q6_K superblock: 128 B ql + 64 B qh uniform, 16 int8 scales uniform in
 * [-32, 31], fp16 d = |N(0, sigma_d)|. */
void levo_synth_q6_k(uint64_t seed, float sigma_d, uint8_t *out, size_t nblocks) {
    uint64_t s = seed;
    for (size_t b = 0; b < nblocks; b++) {
        uint8_t *blk = out + b * 210;
        fill_bytes(&s, blk, 192);
        for (int i = 0; i < 16; i++)
            blk[192 + i] = (uint8_t)(int8_t)((int)(levo_splitmix64_next(&s) % 64) - 32);
        uint16_t h = abs_normal_f16(&s, sigma_d);
        blk[208] = (uint8_t)(h & 0xFF);
        blk[209] = (uint8_t)(h >> 8);
    }
}

/* Q4_K superblock: fp16 d and dmin = |N(0, sigma_d)|, 12 packed scale/min
 * bytes and 128 code bytes uniform. */
void levo_synth_q4_k(uint64_t seed, float sigma_d, uint8_t *out, size_t nblocks) {
    uint64_t s = seed;
    for (size_t b = 0; b < nblocks; b++) {
        uint8_t *blk = out + b * 144;
        uint16_t h = abs_normal_f16(&s, sigma_d);
        blk[0] = (uint8_t)(h & 0xFF);
        blk[1] = (uint8_t)(h >> 8);
        h = abs_normal_f16(&s, sigma_d);
        blk[2] = (uint8_t)(h & 0xFF);
        blk[3] = (uint8_t)(h >> 8);
        fill_bytes(&s, blk + 4, 140);
    }
}

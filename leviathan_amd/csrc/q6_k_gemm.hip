// Q6_K prefill GEMM on the gfx950 matrix cores:  Y[t][r] = sum_k X[t][k] W[r][k].
//
// Stands in for the cooperative-matrix "q6k gemm blocked" kernel
// (lev-forge/src/coopmat.rs:333-425; caller lev-model/src/gpu.rs:345-355).  As
// there, W is dequantised to fp16 -- (d*sc) * (q-32) in f32, then
// round-to-nearest-even -- and X arrives as fp16; products accumulate in f32.
//
// One workgroup = 128 rows x 256 tokens, eight waves in a 2 x 4 arrangement;
// a wave owns 64 rows x 64 tokens = four 32x32 accumulator tiles
// (v_mfma_f32_32x32x16_f16, A = X, B = W^T: lane l holds output row l%32, so
// the stores of Y run along rows).  The wide token tile is what keeps the
// decode (done once per workgroup and K-step) below the matrix-core time.
// K advances by 64 = one nibble plane of half a superblock: the low nibbles of
// a half are its elements 0..63, the high nibbles 64..127, so a thread keeps
// its 32-weight unit (16 ql bytes, 16 qh bytes, scales, d) for two steps.  Per
// step
//   - W: thread (row = tid/4, unit tid%4) decodes 16 weights straight from the
//     2-byte aligned GGUF bytes into fp16 and writes them to LDS, row-major in
//     k with 16 bytes of padding per row;
//   - X: 256 tokens x 128 bytes, eight lanes per token row, to LDS in the same
//     row-major layout;
//   - two LDS buffers: while one is multiplied the other is filled, one
//     barrier per step; operands are requested two steps before they are
//     written to LDS (two register sets), so that a request has two multiply
//     phases to arrive.
// Every lane's fragment is 8 consecutive k (16 bytes) of its row, for both
// operands, so the natural k order is kept.
#include "lev_common.hpp"

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kTR = 128;                 // rows per workgroup
constexpr int kTT = 256;                 // tokens per workgroup (128 measured 6 % slower at 512 tokens)
constexpr int kTK = 64;                  // K-step: one nibble plane of a half superblock
constexpr int kRowHalfs = kTK + 8;       // LDS row: 64 fp16 + 16 bytes of padding
constexpr int kBufHalfs = (kTR + kTT) * kRowHalfs;        // one buffer: W rows, then X rows
constexpr int kGThreads = 2 * kTT;       // one wave per 64 rows x 64 tokens
constexpr int kXLoads = kTT * kTK * 2 / 16 / kGThreads;   // 16-byte loads of X per thread and step
static_assert(kGThreads == kTR * 4, "one 32-weight unit per thread and half");

struct __attribute__((packed, aligned(2))) u32x4_a2 { uint32_t v[4]; };
struct __attribute__((packed, aligned(2))) u32x2_a2 { uint32_t v[2]; };

// One 32-weight unit of a half (Q6.swift:4-62): unit v owns ql[16v..16v+15] of
// the half -- low nibbles are elements 16v+i, high nibbles 64+16v+i -- and the
// qh bytes 16(v&1)..+15 with bit pairs 2(v>>1) (low set) and 2(v>>1)+4 (high
// set); sub-scales (v&1)+2(v>>1) and +4.
struct q6g_unit {
    uint32_t ql[4], qh[4], sc[2], d;
};

__device__ __forceinline__ void q6g_load(const uint8_t *blk, uint32_t half, uint32_t v, q6g_unit &u) {
    u32x4_a2 a = *reinterpret_cast<const u32x4_a2 *>(blk + 64u * half + 16u * v);
    u32x4_a2 b = *reinterpret_cast<const u32x4_a2 *>(blk + 128u + 32u * half + 16u * (v & 1u));
    u32x2_a2 c = *reinterpret_cast<const u32x2_a2 *>(blk + 192u + 8u * half);
    u.d = *reinterpret_cast<const uint16_t *>(blk + 208u);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        u.ql[i] = a.v[i];
        u.qh[i] = b.v[i];
    }
    u.sc[0] = c.v[0];
    u.sc[1] = c.v[1];
}

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

// Four codes packed in `c` -> fp16 weights out[at..at+3]: ds * (q - 32) in f32,
// rounded once to fp16.  The f32 product is formed as fma(q, ds, -32*ds): the
// fused operation rounds the exact q*ds - 32*ds = (q-32)*ds once, which is the
// rounded product itself (-32*ds is exact), and it takes the code byte as it
// stands (byte -> float conversion, no integer subtraction).
__device__ __forceinline__ void q6g_put4(uint32_t c, float ds, float nb, f16x8 &out, int at) {
    f32x2 lo, hi;
    lo.x = fmaf((float)(c & 0xFFu), ds, nb);
    lo.y = fmaf((float)((c >> 8) & 0xFFu), ds, nb);
    hi.x = fmaf((float)((c >> 16) & 0xFFu), ds, nb);
    hi.y = fmaf((float)(c >> 24), ds, nb);
    const f16x2 l16 = __builtin_convertvector(lo, f16x2), h16 = __builtin_convertvector(hi, f16x2);
    out[at + 0] = l16.x;
    out[at + 1] = l16.y;
    out[at + 2] = h16.x;
    out[at + 3] = h16.y;
}

// Decodes one of the unit's two 16-weight groups: HIGH = false -> elements
// 16v.. (low nibbles), true -> 64+16v.. (high nibbles) of the half.
template <bool HIGH>
__device__ __forceinline__ void q6g_decode(const q6g_unit &u, uint32_t v, f16x8 out[2]) {
    const uint32_t pair = v >> 1;
    const uint32_t bi = (v & 1u) + 2u * pair;
    const float d = lev_f16_bits_to_f32(u.d);
    const float ds = d * (float)(int)__builtin_amdgcn_sbfe((int)u.sc[HIGH ? 1 : 0], 8u * bi, 8u);
    const float nb = -32.0f * ds;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t q = u.ql[i], h = u.qh[i];
        const uint32_t c = HIGH ? (((q >> 4) & 0x0F0F0F0Fu) | ((h >> (2u * pair)) & 0x30303030u))
                                : ((q & 0x0F0F0F0Fu) | ((h << (4u - 2u * pair)) & 0x30303030u));
        q6g_put4(c, ds, nb, out[i >> 1], 4 * (i & 1));
    }
}

__global__ void __launch_bounds__(kGThreads)
q6_k_gemm_kernel(const uint8_t *__restrict__ w, const uint16_t *__restrict__ x, float *__restrict__ y,
                 uint32_t in_dim, uint32_t rows, uint32_t tokens) {
    extern __shared__ _Float16 lds[];
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t lr = lane & 31u, lh = lane >> 5;
    const uint32_t wr = wave & 1u, wt = wave >> 1;   // 2 x 4 waves
    const uint32_t row0 = blockIdx.x * kTR, tok0 = blockIdx.y * kTT;
    const uint32_t bpr = in_dim / 256u, halves = in_dim / 128u;

    // decode role: unit dv of the current half of row drow
    const uint32_t drow = tid >> 2, dv = tid & 3u;
    const uint32_t wrow = min(row0 + drow, rows - 1u);   // rows past the end repeat the last one
    const uint8_t *wrow_p = w + (uint64_t)wrow * bpr * 210u;
    // X role: 16-byte piece i = tid + 512*j of the step: token i/8, piece i%8
    const uint16_t *xrow_p[kXLoads];
    uint32_t xdst[kXLoads];
#pragma unroll
    for (int j = 0; j < kXLoads; ++j) {
        const uint32_t i = tid + (uint32_t)j * kGThreads;
        const uint32_t t = min(tok0 + (i >> 3), tokens - 1u);
        xrow_p[j] = x + (uint64_t)t * in_dim + 8u * (i & 7u);
        xdst[j] = kTR * kRowHalfs + (i >> 3) * kRowHalfs + 8u * (i & 7u);
    }
    const uint32_t wdst = drow * kRowHalfs + 16u * dv;

    // Two register sets per operand: what is requested now is parked two steps
    // later, so a request has two multiply phases to arrive.
    q6g_unit Ucur, Unext;
    lev_u32x4 XE[kXLoads], XO[kXLoads];   // activations of even / odd K-steps
    const uint32_t steps = 2u * halves;
    auto request_w = [&](uint32_t half, q6g_unit &U) {
        half = half < halves ? half : halves - 1u;   // past the end: the last half again, never used
        q6g_load(wrow_p + (uint64_t)(half >> 1) * 210u, half & 1u, dv, U);
    };
    auto request_x = [&](uint32_t ks, lev_u32x4 (&XR)[kXLoads]) {
        ks = ks < steps ? ks : steps - 1u;
#pragma unroll
        for (int j = 0; j < kXLoads; ++j)
            XR[j] = *reinterpret_cast<const lev_u32x4 *>(xrow_p[j] + (uint64_t)ks * kTK);
    };
    auto park = [&](_Float16 *buf, const f16x8 wv[2], const lev_u32x4 (&XR)[kXLoads]) {
        *reinterpret_cast<f16x8 *>(buf + wdst) = wv[0];
        *reinterpret_cast<f16x8 *>(buf + wdst + 8) = wv[1];
#pragma unroll
        for (int j = 0; j < kXLoads; ++j) *reinterpret_cast<lev_u32x4 *>(buf + xdst[j]) = XR[j];
    };

    f32x16 acc[2][2];
#pragma unroll
    for (int r = 0; r < 2; ++r)
#pragma unroll
        for (int m = 0; m < 2; ++m)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[r][m][i] = 0.f;

    const uint32_t a_off = kTR * kRowHalfs + (64u * wt + lr) * kRowHalfs + 8u * lh;
    const uint32_t b_off = (64u * wr + lr) * kRowHalfs + 8u * lh;
    auto multiply = [&](const _Float16 *buf) {
#pragma unroll
        for (int kk = 0; kk < kTK / 16; ++kk) {
            f16x8 a[2], b[2];
#pragma unroll
            for (int m = 0; m < 2; ++m)
                a[m] = *reinterpret_cast<const f16x8 *>(buf + a_off + m * 32 * kRowHalfs + 16 * kk);
#pragma unroll
            for (int r = 0; r < 2; ++r)
                b[r] = *reinterpret_cast<const f16x8 *>(buf + b_off + r * 32 * kRowHalfs + 16 * kk);
#pragma unroll
            for (int r = 0; r < 2; ++r)
#pragma unroll
                for (int m = 0; m < 2; ++m)
                    acc[r][m] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[m], b[r], acc[r][m], 0, 0, 0);
        }
    };

    _Float16 *buf0 = lds, *buf1 = lds + kBufHalfs;
    f16x8 wv[2];
    request_w(0, Ucur);
    request_x(0, XE);
    request_x(1, XO);
    request_w(1, Unext);
    q6g_decode<false>(Ucur, dv, wv);
    park(buf0, wv, XE);
    request_x(2, XE);
    __syncthreads();
    // Two K-steps per half: the low-nibble groups (elements 0..63 of the half)
    // from buffer 0, then the high-nibble groups (64..127) from buffer 1.  While
    // a buffer is multiplied the other one is filled, so one barrier a step is
    // enough.  Requests are unconditional (a branch around the loads would make
    // the compiler wait for them at its end) and fenced against the scheduler,
    // which would otherwise move them next to their first use.
    for (uint32_t hf = 0; hf < halves; ++hf) {
        multiply(buf0);                               // step 2hf
        q6g_decode<true>(Ucur, dv, wv);
        park(buf1, wv, XO);                           // -> step 2hf+1
        __builtin_amdgcn_sched_barrier(0);
        request_x(2u * hf + 3u, XO);
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();
        multiply(buf1);                               // step 2hf+1
        q6g_decode<false>(Unext, dv, wv);
        park(buf0, wv, XE);                           // -> step 2hf+2
        Ucur = Unext;
        __builtin_amdgcn_sched_barrier(0);
        request_x(2u * hf + 4u, XE);
        request_w(hf + 2u, Unext);
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();
    }

    // acc[r][m][i]: row 64wr + 32r + lr, token 64wt + 32m + 8(i/4) + 4lh + i%4
#pragma unroll
    for (int r = 0; r < 2; ++r) {
        const uint32_t my_row = row0 + 64u * wr + 32u * r + lr;
        if (my_row >= rows) continue;
#pragma unroll
        for (int m = 0; m < 2; ++m)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const uint32_t t = tok0 + 64u * wt + 32u * m + 8u * (i / 4) + 4u * lh + (i % 4);
                if (t < tokens) y[(uint64_t)t * rows + my_row] = acc[r][m][i];
            }
    }
}

}  // namespace

hipError_t lev_q6_k_gemm_launch(lev_ctx *ctx, const uint8_t *w, const uint16_t *x, float *y,
                                uint32_t in_dim, uint32_t rows, uint32_t tokens) {
    static bool attr_set = false;
    const size_t lds = (size_t)2 * kBufHalfs * sizeof(_Float16);
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&q6_k_gemm_kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    dim3 grid((rows + kTR - 1) / kTR, (tokens + kTT - 1) / kTT);
    hipLaunchKernelGGL(q6_k_gemm_kernel, grid, dim3(kGThreads), lds, ctx->stream, w, x, y, in_dim,
                       rows, tokens);
    return hipGetLastError();
}

extern "C" int lev_hip_q6_k_gemm_prefill(lev_ctx *ctx, const void *d_w, size_t w_bytes,
                                         uint64_t w_off, const uint16_t *d_x_f16, size_t x_count,
                                         float *d_y, size_t y_capacity, uint32_t in_dim,
                                         uint32_t rows, uint32_t tokens) {
    LEV_REQUIRE_CTX(ctx);
    if (tokens == 0 || tokens > (1u << 20))
        return lev_fail(ctx, LEV_ERR_BAD_DIMENSIONS, "q6_k_gemm_prefill: %u tokens", tokens);
    lev_geom g;
    int st = lev_check_matvec(ctx, "q6_k_gemm_prefill", 256, 210, d_w, w_bytes, w_off, d_x_f16,
                              x_count, (uint64_t)in_dim * tokens, d_y, y_capacity,
                              (uint64_t)rows * tokens, in_dim, rows, &g);
    if (st != LEV_OK) return st;
    const uint8_t *w = static_cast<const uint8_t *>(d_w) + w_off;
    if ((reinterpret_cast<uintptr_t>(w) & 1u) || (reinterpret_cast<uintptr_t>(d_x_f16) & 15u))
        return lev_fail(ctx, LEV_ERR_BAD_DIMENSIONS,
                        "q6_k_gemm_prefill: weights must be 2-byte and x 16-byte aligned");
    return lev_hip_check(ctx, lev_q6_k_gemm_launch(ctx, w, d_x_f16, d_y, in_dim, rows, tokens),
                         "q6_k_gemm_prefill launch");
}

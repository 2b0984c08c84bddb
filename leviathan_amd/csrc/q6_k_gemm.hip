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
// K advances by 128 = one half of a superblock.  Per step
//   - W: thread (row = tid/4, one of the half's four 32-weight units) decodes
//     32 weights straight from global memory (2-byte aligned 16-byte runs, as
//     the GGUF layout has them) into fp16 and writes them to LDS, row-major in
//     k with 16 bytes of padding per row;
//   - X: 256 tokens x 256 bytes, sixteen lanes per token row, to LDS in the
//     same row-major layout;
//   - the operands of step ks+1 are requested before the MFMAs of step ks and
//     written to LDS after them (registers in between, two barriers a step).
// Every lane's fragment is 8 consecutive k (16 bytes) of its row, for both
// operands, so the natural k order is kept.
#include "lev_common.hpp"

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kTR = 128;                 // rows per workgroup
constexpr int kTT = 256;                 // tokens per workgroup (128 measured 6 % slower at 512 tokens)
constexpr int kTK = 128;                 // K-step
constexpr int kRowHalfs = kTK + 8;       // LDS row: 128 fp16 + 16 bytes of padding
constexpr int kGThreads = 2 * kTT;       // one wave per 64 rows x 64 tokens
constexpr int kUnits = kTR * 4 / kGThreads;               // 32-weight units decoded per thread and step
constexpr int kXLoads = kTT * kTK * 2 / 16 / kGThreads;   // 16-byte loads of X per thread and step

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

// Decodes the unit into its two 16-weight groups: lo = elements 16v.., hi = 64+16v..
__device__ __forceinline__ void q6g_decode(const q6g_unit &u, uint32_t v, f16x8 lo[2], f16x8 hi[2]) {
    const uint32_t pair = v >> 1;
    const uint32_t shl = 4u - 2u * pair, shr = 2u * pair;
    const uint32_t bi = (v & 1u) + 2u * pair;
    const float d = lev_f16_bits_to_f32(u.d);
    const float ds_lo = d * (float)(int)__builtin_amdgcn_sbfe((int)u.sc[0], 8u * bi, 8u);
    const float ds_hi = d * (float)(int)__builtin_amdgcn_sbfe((int)u.sc[1], 8u * bi, 8u);
    const float nb_lo = -32.0f * ds_lo, nb_hi = -32.0f * ds_hi;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t q = u.ql[i], h = u.qh[i];
        const uint32_t cl = (q & 0x0F0F0F0Fu) | ((h << shl) & 0x30303030u);
        const uint32_t ch = ((q >> 4) & 0x0F0F0F0Fu) | ((h >> shr) & 0x30303030u);
        q6g_put4(cl, ds_lo, nb_lo, lo[i >> 1], 4 * (i & 1));
        q6g_put4(ch, ds_hi, nb_hi, hi[i >> 1], 4 * (i & 1));
    }
}

__global__ void __launch_bounds__(kGThreads)
q6_k_gemm_kernel(const uint8_t *__restrict__ w, const uint16_t *__restrict__ x, float *__restrict__ y,
                 uint32_t in_dim, uint32_t rows, uint32_t tokens) {
    extern __shared__ _Float16 lds[];
    _Float16 *wsh = lds;                          // [kTR][kRowHalfs]
    _Float16 *xsh = lds + kTR * kRowHalfs;        // [kTT][kRowHalfs]
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t lr = lane & 31u, lh = lane >> 5;
    const uint32_t wr = wave & 1u, wt = wave >> 1;   // 2 x kTT/64 waves
    const uint32_t row0 = blockIdx.x * kTR, tok0 = blockIdx.y * kTT;
    const uint32_t bpr = in_dim / 256u, steps = in_dim / kTK;

    // decode role: kUnits consecutive units of the step's half of one row
    const uint32_t drow = tid / (4u / kUnits), dv = kUnits * (tid % (4u / kUnits));
    const uint32_t wrow = min(row0 + drow, rows - 1u);   // rows past the end repeat the last one
    const uint8_t *wrow_p = w + (uint64_t)wrow * bpr * 210u;
    // X role: 16-byte piece i = tid + 256*j of the step: token i/16, piece i%16
    const uint16_t *xrow_p[kXLoads];
#pragma unroll
    for (int j = 0; j < kXLoads; ++j) {
        const uint32_t i = tid + (uint32_t)j * kGThreads;
        const uint32_t t = min(tok0 + (i >> 4), tokens - 1u);
        xrow_p[j] = x + (uint64_t)t * in_dim + 8u * (i & 15u);
    }

    q6g_unit U[kUnits];
    lev_u32x4 XR[kXLoads];
    auto request = [&](uint32_t ks) {
        const uint8_t *blk = wrow_p + (uint64_t)(ks >> 1) * 210u;
#pragma unroll
        for (int k = 0; k < kUnits; ++k) q6g_load(blk, ks & 1u, dv + k, U[k]);
#pragma unroll
        for (int j = 0; j < kXLoads; ++j)
            XR[j] = *reinterpret_cast<const lev_u32x4 *>(xrow_p[j] + (uint64_t)ks * kTK);
    };
    auto park = [&]() {
#pragma unroll
        for (int k = 0; k < kUnits; ++k) {
            f16x8 lo[2], hi[2];
            q6g_decode(U[k], dv + k, lo, hi);
            _Float16 *dst = wsh + drow * kRowHalfs + 16u * (dv + k);
            *reinterpret_cast<f16x8 *>(dst) = lo[0];
            *reinterpret_cast<f16x8 *>(dst + 8) = lo[1];
            *reinterpret_cast<f16x8 *>(dst + 64) = hi[0];
            *reinterpret_cast<f16x8 *>(dst + 72) = hi[1];
        }
#pragma unroll
        for (int j = 0; j < kXLoads; ++j) {
            const uint32_t i = tid + (uint32_t)j * kGThreads;
            *reinterpret_cast<lev_u32x4 *>(xsh + (i >> 4) * kRowHalfs + 8u * (i & 15u)) = XR[j];
        }
    };

    f32x16 acc[2][2];
#pragma unroll
    for (int r = 0; r < 2; ++r)
#pragma unroll
        for (int m = 0; m < 2; ++m)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[r][m][i] = 0.f;

    request(0);
    park();
    __syncthreads();
    const _Float16 *a_base = xsh + (64u * wt + lr) * kRowHalfs + 8u * lh;
    const _Float16 *b_base = wsh + (64u * wr + lr) * kRowHalfs + 8u * lh;
    for (uint32_t ks = 0; ks < steps; ++ks) {
        // the next step's operands are requested unconditionally (the last step
        // asks for its own again): a branch around the loads would make the
        // compiler wait for them at its end
        request(ks + 1u < steps ? ks + 1u : ks);
#pragma unroll
        for (int kk = 0; kk < kTK / 16; ++kk) {
            f16x8 a[2], b[2];
#pragma unroll
            for (int m = 0; m < 2; ++m)
                a[m] = *reinterpret_cast<const f16x8 *>(a_base + m * 32 * kRowHalfs + 16 * kk);
#pragma unroll
            for (int r = 0; r < 2; ++r)
                b[r] = *reinterpret_cast<const f16x8 *>(b_base + r * 32 * kRowHalfs + 16 * kk);
#pragma unroll
            for (int r = 0; r < 2; ++r)
#pragma unroll
                for (int m = 0; m < 2; ++m)
                    acc[r][m] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[m], b[r], acc[r][m], 0, 0, 0);
        }
        __syncthreads();   // every wave is done reading this step's tiles
        if (ks + 1u < steps) park();
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
    const size_t lds = (size_t)(kTR + kTT) * kRowHalfs * sizeof(_Float16);
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

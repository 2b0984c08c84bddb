// Q4_K prefill GEMM on the gfx950 matrix cores:  Y[t][r] = sum_k X[t][k] W[r][k].
//
// Stands in for the cooperative-matrix "q4k gemm blocked" kernel
// (lev-forge/src/coopmat.rs:236-323; caller lev-model/src/gpu.rs:345-355;
// gate lev-cli/src/main.rs:1187-1279).  As there, W is dequantised to fp16
// (f32 arithmetic d*sc*q - dmin*m, then round-to-nearest-even) and X arrives
// as fp16; products accumulate in f32.  Both operands use the same 16-bit type
// because one MFMA takes one input type; fp16 keeps X exactly as given.
//
// Tiling (one workgroup = 4 waves = 256 tokens x 128 rows):
//   - wave w owns rows 32w..32w+31 of the tile for ALL 256 tokens: 8
//     accumulator tiles of 32x32 (v_mfma_f32_32x32x16_f16), A = X, B = W^T, so
//     lane l holds output row (l%32) -> stores of Y are contiguous along rows;
//   - W never goes through LDS: lane (r = l%32, h = l/32) loads the 16 code
//     bytes 16h..16h+15 of each 32-byte chunk of ITS row plus the superblock
//     header and dequantises them in registers straight into B fragments, so
//     every weight is decoded exactly once per workgroup;
//   - X goes through LDS in K-steps of 64 (one Q4_K chunk: sub-blocks 2c, 2c+1),
//     double-buffered, rows padded to 144 bytes so that the 128-bit fragment
//     reads of 8 consecutive lanes cover all 32 banks.
// K order inside a 64-step is permuted consistently on both operands:
// MFMA q (0..3) of chunk c takes, for lane half h, elements
//   q<2 : 64c + 16h + 8q .. +7        (low nibbles of code bytes 8q..8q+7)
//   q>=2: 64c + 32 + 16h + 8(q-2) ..  (high nibbles of the same bytes)
#include "lev_common.hpp"

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kThreads = 256;
constexpr int kBM = 256;          // tokens per workgroup
constexpr int kBN = 128;          // rows per workgroup (32 per wave)
constexpr int kMT = kBM / 32;     // accumulator tiles per wave
constexpr int kKS = 64;           // K-step
constexpr int kXRow = 144;        // bytes per token row in LDS (128 + 16 pad)
constexpr int kXBuf = kBM * kXRow;

// (d*sc, dmin*m) of the 8 sub-blocks of a superblock (lev-cpu/src/lib.rs:64-74,
// 117-124).
__device__ __forceinline__ void q4k_all_factors(const lev_u32x4 hdr, float d1[8], float mm[8]) {
    const float d = lev_f16_bits_to_f32(hdr.x & 0xFFFFu);
    const float dmin = lev_f16_bits_to_f32(hdr.x >> 16);
    const uint32_t s03 = hdr.y, s47 = hdr.z, s811 = hdr.w;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        uint32_t sc = (s03 >> (8 * j)) & 63u, mn = (s47 >> (8 * j)) & 63u;
        d1[j] = d * (float)sc;
        mm[j] = dmin * (float)mn;
        uint32_t a = (s811 >> (8 * j)) & 0xFFu;
        uint32_t sc2 = (a & 0x0Fu) | (((s03 >> (8 * j + 6)) & 3u) << 4);
        uint32_t mn2 = (a >> 4) | (((s47 >> (8 * j + 6)) & 3u) << 4);
        d1[4 + j] = d * (float)sc2;
        mm[4 + j] = dmin * (float)mn2;
    }
}

// One weight exactly as the reference rounds it: f32(d1*q - mm) first, THEN
// round-to-nearest-even to fp16 (dequant_block_f32 followed by f32_to_f16_bits,
// lev-cli/src/main.rs:1201-1217).  The empty asm pins the f32 value in a
// register so that the compiler cannot merge the multiply-add with the
// conversion into a single-rounding mixed-precision FMA, which differs from
// the two-step rounding in about one weight in ten thousand.
__device__ __forceinline__ _Float16 q4k_weight_f16(float d1, float code, float mm) {
    float w32 = fmaf(d1, code, -mm);   // d1*code is exact (17 + 4 bits): one rounding, as in the reference
    asm volatile("" : "+v"(w32));
    return (_Float16)w32;
}

// 8 weights (one per code byte of the two dwords, nibble selected by `hi`)
// -> fp16 B fragment, bit-exact with fp16(f32(d1*q - mm)).
__device__ __forceinline__ f16x8 q4k_frag(uint32_t q0, uint32_t q1, bool hi, float d1, float mm) {
    uint32_t a = hi ? (q0 >> 4) : q0, b = hi ? (q1 >> 4) : q1;
    a &= 0x0F0F0F0Fu;
    b &= 0x0F0F0F0Fu;
    f16x8 f;
    f[0] = q4k_weight_f16(d1, (float)(a & 0xFFu), mm);
    f[1] = q4k_weight_f16(d1, (float)((a >> 8) & 0xFFu), mm);
    f[2] = q4k_weight_f16(d1, (float)((a >> 16) & 0xFFu), mm);
    f[3] = q4k_weight_f16(d1, (float)(a >> 24), mm);
    f[4] = q4k_weight_f16(d1, (float)(b & 0xFFu), mm);
    f[5] = q4k_weight_f16(d1, (float)((b >> 8) & 0xFFu), mm);
    f[6] = q4k_weight_f16(d1, (float)((b >> 16) & 0xFFu), mm);
    f[7] = q4k_weight_f16(d1, (float)(b >> 24), mm);
    return f;
}

// grid (ceil(rows/128), ceil(tokens/256)); LDS 2*kXBuf bytes.
__global__ void __launch_bounds__(kThreads)
q4_k_gemm_kernel(const uint8_t *__restrict__ w, const uint16_t *__restrict__ x,
                 float *__restrict__ y, uint32_t in_dim, uint32_t rows, uint32_t tokens) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t lr = lane & 31u, lh = lane >> 5;
    const uint32_t row0 = blockIdx.x * kBN + wave * 32u;
    const uint32_t tok0 = blockIdx.y * kBM;
    const uint32_t nsb = in_dim / 256u;
    const uint32_t my_row = row0 + lr;
    const uint8_t *wrow = w + (uint64_t)(my_row < rows ? my_row : rows - 1u) * nsb * 144u;

    // X staging: thread covers 16 bytes of 8 token rows per K-step.
    const uint32_t xs_tok = tid >> 3;          // 0..31, + 32*i
    const uint32_t xs_col = (tid & 7u) * 16u;  // byte offset inside the 128-byte K-step row
    lev_u32x4 xr[8];
    auto x_load = [&](uint32_t kstep) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            uint32_t t = tok0 + xs_tok + 32u * i;
            if (t < tokens)
                xr[i] = *reinterpret_cast<const lev_u32x4 *>(
                    reinterpret_cast<const uint8_t *>(x) + ((uint64_t)t * in_dim + kstep * kKS) * 2u + xs_col);
            else
                xr[i] = lev_u32x4{0u, 0u, 0u, 0u};
        }
    };
    auto x_store = [&](uint32_t buf) {
#pragma unroll
        for (int i = 0; i < 8; ++i)
            *reinterpret_cast<lev_u32x4 *>(lds + buf * kXBuf + (xs_tok + 32u * i) * kXRow + xs_col) = xr[i];
    };

    f32x16 acc[kMT];
#pragma unroll
    for (int m = 0; m < kMT; ++m)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[m][i] = 0.f;

    const uint32_t nsteps = nsb * 4u;
    x_load(0);
    x_store(0);
    __syncthreads();

    for (uint32_t sb = 0; sb < nsb; ++sb) {
        const uint8_t *blk = wrow + (uint64_t)sb * 144u;
        lev_u32x4 hdr = *reinterpret_cast<const lev_u32x4 *>(blk);
        lev_u32x4 qs[4];
#pragma unroll
        for (int cc = 0; cc < 4; ++cc)
            qs[cc] = *reinterpret_cast<const lev_u32x4 *>(blk + 16u + 32u * cc + 16u * lh);
        float d1[8], mm[8];
        q4k_all_factors(hdr, d1, mm);
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const uint32_t ks = sb * 4u + c;
            if (ks + 1 < nsteps) x_load(ks + 1);

            // this lane's 32 weights of chunk c -> four B fragments
            const lev_u32x4 q = qs[c];
            f16x8 bf[4];
            bf[0] = q4k_frag(q.x, q.y, false, d1[2 * c], mm[2 * c]);
            bf[1] = q4k_frag(q.z, q.w, false, d1[2 * c], mm[2 * c]);
            bf[2] = q4k_frag(q.x, q.y, true, d1[2 * c + 1], mm[2 * c + 1]);
            bf[3] = q4k_frag(q.z, q.w, true, d1[2 * c + 1], mm[2 * c + 1]);

            const uint8_t *xb = lds + (ks & 1u) * kXBuf + lr * kXRow + 32u * lh;
#pragma unroll
            for (int qq = 0; qq < 4; ++qq) {
                // byte offset of this MFMA's 8 activations inside the 128-byte row
                const uint32_t koff = (qq < 2 ? 16u * qq : 64u + 16u * (qq - 2));
#pragma unroll
                for (int m = 0; m < kMT; ++m) {
                    f16x8 a = *reinterpret_cast<const f16x8 *>(xb + m * 32 * kXRow + koff);
                    acc[m] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, bf[qq], acc[m], 0, 0, 0);
                }
            }
            if (ks + 1 < nsteps) x_store((ks + 1) & 1u);
            __syncthreads();
        }
    }

    // D layout of the 32x32 tile: lane -> column n = l%32 (our row), register
    // i -> line m = 8*(i/4) + 4*(l/32) + i%4 (our token).
    if (my_row < rows) {
#pragma unroll
        for (int m = 0; m < kMT; ++m)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                uint32_t t = tok0 + m * 32 + 8 * (i / 4) + 4 * lh + (i % 4);
                if (t < tokens) y[(uint64_t)t * rows + my_row] = acc[m][i];
            }
    }
}

}  // namespace

hipError_t lev_q4_k_gemm_launch(lev_ctx *ctx, const uint8_t *w, const uint16_t *x, float *y,
                                uint32_t in_dim, uint32_t rows, uint32_t tokens) {
    static bool attr_set = false;
    const size_t lds = 2 * (size_t)kXBuf;
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&q4_k_gemm_kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    dim3 grid((rows + kBN - 1) / kBN, (tokens + kBM - 1) / kBM);
    hipLaunchKernelGGL(q4_k_gemm_kernel, grid, dim3(kThreads), lds, ctx->stream, w, x, y, in_dim,
                       rows, tokens);
    return hipGetLastError();
}

extern "C" int lev_hip_q4_k_gemm_prefill(lev_ctx *ctx, const void *d_w, size_t w_bytes,
                                         uint64_t w_off, const uint16_t *d_x_f16, size_t x_count,
                                         float *d_y, size_t y_capacity, uint32_t in_dim,
                                         uint32_t rows, uint32_t tokens) {
    LEV_REQUIRE_CTX(ctx);
    if (tokens == 0 || tokens > (1u << 20))
        return lev_fail(ctx, LEV_ERR_BAD_DIMENSIONS, "q4_k_gemm_prefill: %u tokens", tokens);
    lev_geom g;
    int st = lev_check_matvec(ctx, "q4_k_gemm_prefill", 256, 144, d_w, w_bytes, w_off, d_x_f16,
                              x_count, (uint64_t)in_dim * tokens, d_y, y_capacity,
                              (uint64_t)rows * tokens, in_dim, rows, &g);
    if (st != LEV_OK) return st;
    const uint8_t *w = static_cast<const uint8_t *>(d_w) + w_off;
    if ((reinterpret_cast<uintptr_t>(w) & 15u) || (reinterpret_cast<uintptr_t>(d_x_f16) & 15u))
        return lev_fail(ctx, LEV_ERR_BAD_DIMENSIONS,
                        "q4_k_gemm_prefill: weights and x must be 16-byte aligned");
    return lev_hip_check(ctx, lev_q4_k_gemm_launch(ctx, w, d_x_f16, d_y, in_dim, rows, tokens),
                         "q4_k_gemm_prefill launch");
}

// Q6_K prefill GEMM on the gfx950 matrix cores:  Y[t][r] = sum_k X[t][k] W[r][k].
//
// Stands in for the cooperative-matrix "q6k gemm blocked" kernel
// (lev-forge/src/coopmat.rs:333-425; caller lev-model/src/gpu.rs:345-355).  As
// there, W is dequantised to fp16 -- (d*sc) * (q-32) in f32, then
// round-to-nearest-even -- and X arrives as fp16; products accumulate in f32.
//
// One workgroup = 128 rows x 256 tokens, eight waves with split roles (the
// arrangement of the Q4_K kernel's X path, carried to the weights as well):
//   - waves 0..3 multiply and do nothing else: wave w owns tokens 64w..64w+63
//     times all 128 rows = 2 x 4 accumulator tiles (v_mfma_f32_32x32x16_f16,
//     A = X, B = W^T: lane l holds output row l%32, so the stores of Y run along
//     rows); per K-step of 64 it reads the X fragments of its tokens and the
//     four row tiles' B fragments from LDS, one read in the shadow of each MFMA,
//     and never waits for global memory;
//   - waves 4..7 feed them: wave 4+i moves a quarter of the step's X with
//     direct global -> LDS loads (XOR-swizzled rows, four buffers, two steps in
//     flight) and, between the requests, decodes row tile i -- lane (row l%32,
//     half h = l/32) owns elements 32h..32h+31 of the step: 32 contiguous ql
//     bytes, one bit pair of 32 qh bytes, two sub-scales -- into four fp16 B
//     fragments of the next step (two buffers).
// K advances by 64 = one nibble plane of half a superblock (the low nibbles of
// a half are its elements 0..63, the high nibbles 64..127).  K order inside a
// step, on both operands: MFMA q (0..3), lane half h takes elements
// 32h + 8q .. +7.  One barrier per step, a bare s_barrier behind counted waits.
#include "lev_common.hpp"

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kTR = 128;                 // rows per workgroup
constexpr int kTT = 256;                 // tokens per workgroup (128 measured 6 % slower at 512 tokens)
constexpr int kTK = 64;                  // K-step: one nibble plane of a half superblock

struct __attribute__((packed, aligned(2))) u32x4_a2 { uint32_t v[4]; };

// Four codes packed in `c` -> fp16 weights out[at..at+3], one instruction per weight
// (Q6.swift:4-62 for the layout).  ds = d * sc has at most 18
// significant bits and q - 32 six, so ds * (q - 32) is exact in f32 and the reference's
// two roundings (f32, then fp16) are one rounding of the exact product.  A code byte
// under the exponent byte 0x64 is the fp16 number 1024 + q; fma(1024 + q, ds, -1056 ds)
// is that exact product, and the mixed-precision FMA rounds it to fp16 once.
__device__ __forceinline__ void q6g_put4_mix(uint32_t c, float ds, float nbm, f16x8 &out, int at) {
    const uint32_t ma = __builtin_amdgcn_perm(0x64646464u, c, 0x04020400u);   // bytes (c0, 0x64, c2, 0x64)
    const uint32_t mb = __builtin_amdgcn_perm(0x64646464u, c, 0x04030401u);   // bytes (c1, 0x64, c3, 0x64)
    const f16x2 a = __builtin_bit_cast(f16x2, ma), b = __builtin_bit_cast(f16x2, mb);
    out[at + 0] = (_Float16)fmaf((float)a.x, ds, nbm);
    out[at + 1] = (_Float16)fmaf((float)b.x, ds, nbm);
    out[at + 2] = (_Float16)fmaf((float)a.y, ds, nbm);
    out[at + 3] = (_Float16)fmaf((float)b.y, ds, nbm);
}

constexpr int kRXRow = 128;                    // bytes per token row in LDS
constexpr int kRXBuf = kTT * kRXRow;           // 32 KB
constexpr int kRXBufs = 4;
constexpr int kRBFrag = 64 * 16;               // one B fragment: 16 bytes per lane
constexpr int kRRT = kTR / 32;                 // row tiles
constexpr int kRBBuf = 4 * kRRT * kRBFrag;     // [q][row tile][lane], one K-step; two of them
constexpr int kRThreads = 512;

#define LEV_Q6G_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 0xF) | (((n) >> 4) << 14) | (7 << 4) | (15 << 8))

__global__ void __launch_bounds__(kRThreads)
q6_k_gemm_kernel(const uint8_t *__restrict__ w, const uint16_t *__restrict__ x, float *__restrict__ y,
                 uint32_t in_dim, uint32_t rows, uint32_t tokens) {
    extern __shared__ __attribute__((aligned(16))) uint8_t ldsr[];
    uint8_t *const ldsb = ldsr + kRXBufs * kRXBuf;
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t lr = lane & 31u, lh = lane >> 5;
    const uint32_t row0 = blockIdx.x * kTR;
    const uint32_t nsb = in_dim / 256u, nsteps = nsb * 4u;
    // A workgroup takes token tiles blockIdx.y, blockIdx.y + gridDim.y, ... of its rows one after the
    // other: the stores that end a tile drain while the next one is multiplied.
    const uint32_t ntt = (tokens + kTT - 1u) / kTT;

    if (wave >= 4u) {
        const uint32_t lw = __builtin_amdgcn_readfirstlane(wave) - 4u, ltok = lane >> 3, lpos = lane & 7u;
        const uint32_t drow = row0 + 32u * lw + lr;
        const uint8_t *const wrow = w + (uint64_t)(drow < rows ? drow : rows - 1u) * nsb * 210u;
        for (uint32_t ty = blockIdx.y; ty < ntt; ty += gridDim.y) {
        const uint32_t tok0 = ty * kTT;
        const uint8_t *const xtile = reinterpret_cast<const uint8_t *>(x) + (uint64_t)tok0 * in_dim * 2u;
        uint32_t voff[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const uint32_t tl = 8u * (8u * lw + j) + ltok;
            const uint32_t t = tok0 + tl < tokens ? tl : tokens - 1u - tok0;
            voff[j] = t * in_dim * 2u + 16u * (lpos ^ (ltok & 7u));
        }
        auto x_request_one = [&](uint32_t kstep, uint32_t buf, int j) {
            const uint8_t *const xk = xtile + (uint64_t)kstep * (kTK * 2u);
            uint8_t *dst = ldsr + buf * kRXBuf + (8u * lw + j) * 1024u;
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(xk + voff[j]),
                                             (__attribute__((address_space(3))) void *)dst, 16, 0, 0);
        };
        // one superblock of the lane's row: ql[hf][8 dwords], qh[hf][8 dwords], 16 sub-scales, d
        struct wregs {
            uint32_t ql[2][8], qh[2][8], sc[4], d;
        };
        wregs Wn, Wc;
        float dsc;
        auto w_load = [&](uint32_t sb) {
            const uint32_t sbc = sb < nsb ? sb : nsb - 1u;
            const uint8_t *blk = wrow + (uint64_t)sbc * 210u;
#pragma unroll
            for (int hf = 0; hf < 2; ++hf)
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    const u32x4_a2 a = *reinterpret_cast<const u32x4_a2 *>(blk + 64u * hf + 32u * lh + 16u * i);
                    const u32x4_a2 b = *reinterpret_cast<const u32x4_a2 *>(blk + 128u + 32u * hf + 16u * i);
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        Wn.ql[hf][4 * i + k] = a.v[k];
                        Wn.qh[hf][4 * i + k] = b.v[k];
                    }
                }
            const u32x4_a2 s4 = *reinterpret_cast<const u32x4_a2 *>(blk + 192u);
#pragma unroll
            for (int k = 0; k < 4; ++k) Wn.sc[k] = s4.v[k];
            Wn.d = *reinterpret_cast<const uint16_t *>(blk + 208u);
        };
        // The hand-over is spelled as moves the compiler may not reorder: a plain copy is
        // free to move up to the request, and the wait for the loads with it.
        auto hand = [&](uint32_t &cur, const uint32_t &next) {
            uint32_t t;
            asm volatile("v_mov_b32 %0, %1" : "=v"(t) : "v"(next));
            cur = t;
        };
        auto take = [&]() {
#pragma unroll
            for (int hf = 0; hf < 2; ++hf)
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    hand(Wc.ql[hf][k], Wn.ql[hf][k]);
                    hand(Wc.qh[hf][k], Wn.qh[hf][k]);
                }
#pragma unroll
            for (int k = 0; k < 4; ++k) hand(Wc.sc[k], Wn.sc[k]);
            hand(Wc.d, Wn.d);
            dsc = lev_f16_bits_to_f32(Wc.d);
        };
        // fragment q of step (hf, np) -> B buffer `buf`
        auto decode_one = [&](int hf, int np, int q, uint32_t buf) {
            const uint32_t sw = Wc.sc[2 * hf + np];
            const float ds = dsc * (float)(int)__builtin_amdgcn_sbfe((int)sw, 8u * (2u * lh + (uint32_t)(q >> 1)), 8u);
            const float nbm = -1056.0f * ds;
            f16x8 f;
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const uint32_t a = Wc.ql[hf][2 * q + i], h = Wc.qh[hf][2 * q + i];
                const uint32_t c = np ? (((a >> 4) & 0x0F0F0F0Fu) | ((h >> (2u * lh)) & 0x30303030u))
                                      : ((a & 0x0F0F0F0Fu) | ((h << (4u - 2u * lh)) & 0x30303030u));
                q6g_put4_mix(c, ds, nbm, f, 4 * i);
            }
            *reinterpret_cast<f16x8 *>(ldsb + buf * kRBBuf + (q * kRRT + lw) * kRBFrag + lane * 16u) = f;
        };
        w_load(0);
        take();
#pragma unroll
        for (int q = 0; q < 4; ++q) decode_one(0, 0, q, 0u);
#pragma unroll
        for (int j = 0; j < 8; ++j) x_request_one(0, 0, j);
#pragma unroll
        for (int j = 0; j < 8; ++j) x_request_one(1 < nsteps ? 1 : nsteps - 1, 1, j);
        // Loads in flight at the barrier of step ks = 4 sb + c, oldest first (they
        // complete in issue order): c = 1: X(ks) W(sb+1) X(ks+1), otherwise
        // X(ks) X(ks+1).  X(ks) has landed once at most 8 (c = 1: 18) newer loads
        // are outstanding.
        for (uint32_t sb = 0; sb < nsb; ++sb) {
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const uint32_t ks = sb * 4u + c;
                if (c == 1)
                    LEV_Q6G_WAIT_VMCNT(18);
                else
                    LEV_Q6G_WAIT_VMCNT(8);
                __builtin_amdgcn_s_waitcnt(0xC07F);   // this wave's B fragments of step ks are in LDS
                asm volatile("s_barrier" ::: "memory");
                __builtin_amdgcn_sched_barrier(0);   // a step's decode stays inside the step
                const uint32_t kx = ks + 2 < nsteps ? ks + 2 : nsteps - 1, bx = (ks + 2) & 3u;
                const int cn = c == 3 ? 0 : c + 1;
                if (c == 0) {   // pinned here: the counts above depend on where these loads are issued
                    __builtin_amdgcn_sched_barrier(0);
                    w_load(sb + 1u);
                    __builtin_amdgcn_sched_barrier(0);
                }
                if (c == 3) take();
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    x_request_one(kx, bx, 2 * q);
                    x_request_one(kx, bx, 2 * q + 1);
                    decode_one(cn >> 1, cn & 1, q, (ks + 1u) & 1u);
                }
            }
        }
        }
        LEV_Q6G_WAIT_VMCNT(0);
        return;
    }

    for (uint32_t ty = blockIdx.y; ty < ntt; ty += gridDim.y) {
    const uint32_t tok0 = ty * kTT;
    f32x16 acc[kRRT][2];
#pragma unroll
    for (int r = 0; r < kRRT; ++r)
#pragma unroll
        for (int m = 0; m < 2; ++m)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[r][m][i] = 0.f;

    // Rotated by two MFMA groups: groups 2 and 3 of a step are multiplied after
    // the barrier of the next step, from fragments read before it, while the
    // first fragments of the new step come in.
    f16x8 a_buf[4][2], b_buf[4][kRRT];
#pragma unroll
    for (int g = 2; g < 4; ++g) {
#pragma unroll
        for (int m = 0; m < 2; ++m)
#pragma unroll
            for (int i = 0; i < 8; ++i) a_buf[g][m][i] = (_Float16)0.f;
#pragma unroll
        for (int r = 0; r < kRRT; ++r)
#pragma unroll
            for (int i = 0; i < 8; ++i) b_buf[g][r][i] = (_Float16)0.f;
    }
    for (uint32_t ks = 0; ks < nsteps; ++ks) {
        __builtin_amdgcn_s_waitcnt(0xC07F);   // the reads of step ks-1 have arrived
        asm volatile("s_barrier" ::: "memory");
        const uint8_t *xb = ldsr + (ks & 3u) * kRXBuf + (wave * 64u + lr) * kRXRow;
        const uint8_t *bb = ldsb + (ks & 1u) * kRBBuf + lane * 16u;
        // fragment `which` (use order a0 b0 b1 b2 b3 a1) of MFMA group q
        auto frag_read_one = [&](int q, int which) {
            if (which == 0 || which == 5) {
                const int m = which == 0 ? 0 : 1;
                const uint32_t koff = 16u * ((4u * lh + (uint32_t)q) ^ (lr & 7u));
                a_buf[q][m] = *reinterpret_cast<const f16x8 *>(xb + m * 32 * kRXRow + koff);
            } else {
                const int r = which - 1;
                b_buf[q][r] = *reinterpret_cast<const f16x8 *>(bb + (q * kRRT + r) * kRBFrag);
            }
        };
#pragma unroll
        for (int f = 0; f < 6; ++f) frag_read_one(0, f);
#pragma unroll
        for (int ph = 0; ph < 4; ++ph) {
            const int q = (ph + 2) & 3;          // the MFMA group of this phase
            const int rg = ph == 0 ? 1 : ph;     // the group read in this phase (none in phase 1)
#pragma unroll
            for (int i = 0; i < 2 * kRRT; ++i) {
                const int r = i % kRRT, m = i / kRRT;
                acc[r][m] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a_buf[q][m], b_buf[q][r], acc[r][m], 0, 0, 0);
                if (ph != 1 && i < 6) frag_read_one(rg, i);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }
#pragma unroll
    for (int g = 2; g < 4; ++g)
#pragma unroll
        for (int i = 0; i < 2 * kRRT; ++i) {
            const int r = i % kRRT, m = i / kRRT;
            acc[r][m] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a_buf[g][m], b_buf[g][r], acc[r][m], 0, 0, 0);
        }

#pragma unroll
    for (int r = 0; r < kRRT; ++r) {
        const uint32_t my_row = row0 + 32u * r + lr;
        if (my_row >= rows) continue;
#pragma unroll
        for (int m = 0; m < 2; ++m)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const uint32_t t = tok0 + wave * 64u + m * 32 + 8 * (i / 4) + 4 * lh + (i % 4);
                if (t < tokens) y[(uint64_t)t * rows + my_row] = acc[r][m][i];
            }
    }
    }
}

}  // namespace

hipError_t lev_q6_k_gemm_launch(lev_ctx *ctx, const uint8_t *w, const uint16_t *x, float *y,
                                uint32_t in_dim, uint32_t rows, uint32_t tokens) {
    static bool attr_set = false;
    const size_t lds = (size_t)kRXBufs * kRXBuf + 2 * kRBBuf;   // 160 KB: one workgroup per CU
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&q6_k_gemm_kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    // One workgroup per CU (160 KB of LDS).  When the row tiles alone nearly fill the chip, a workgroup
    // takes several token tiles of its rows in turn instead of leaving them to a later round of
    // workgroups: as many rounds of work, and only the last tile's stores are not covered
    // (512 x 32000 x 4096: 179.2 us against 181.6).
    const uint32_t nrt = (rows + kTR - 1) / kTR, ntt = (tokens + kTT - 1) / kTT;
    const uint32_t cus = (uint32_t)ctx->props.multiProcessorCount;
    uint32_t gy = ntt;
    if ((uint64_t)nrt * ntt > cus && nrt <= cus) {
        const uint32_t fit = cus / nrt;                                  // token tiles side by side in one round
        const uint32_t turns = (ntt + fit - 1) / fit;                    // tiles a workgroup then takes in turn
        const uint64_t rounds = ((uint64_t)nrt * ntt + cus - 1) / cus;   // rounds of one-tile workgroups
        if (turns <= rounds) gy = fit < ntt ? fit : ntt;
    }

    dim3 grid(nrt, gy);
    hipLaunchKernelGGL(q6_k_gemm_kernel, grid, dim3(kRThreads), lds, ctx->stream, w, x, y, in_dim,
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
    if (in_dim > (1u << 22))   // the X loaders keep 32-bit byte offsets inside a 256-token tile
        return lev_fail(ctx, LEV_ERR_BAD_DIMENSIONS, "q6_k_gemm_prefill: in_dim %u above 4194304", in_dim);
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

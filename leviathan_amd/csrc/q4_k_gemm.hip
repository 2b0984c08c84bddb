// Q4_K prefill GEMM on the gfx950 matrix cores:  Y[t][r] = sum_k X[t][k] W[r][k].
//
// Stands in for the cooperative-matrix "q4k gemm blocked" kernel
// (lev-forge/src/coopmat.rs:236-323; caller lev-model/src/gpu.rs:345-355;
// gate lev-cli/src/main.rs:1187-1279).  As there, W is dequantised to fp16
// (f32 arithmetic d*sc*q - dmin*m, then round-to-nearest-even) and X arrives
// as fp16; products accumulate in f32.  Both operands use the same 16-bit type
// because one MFMA takes one input type; fp16 keeps X exactly as given.
//
// One workgroup = 256 tokens x 96 rows, so that 512 x 12288 makes 256 workgroups,
// one per CU.  Eight waves:
//   - waves 0..3 multiply.  Wave w owns tokens 64w..64w+63 (two 32-token tiles)
//     times all 96 rows (three 32-row tiles): 6 accumulator tiles of 32x32
//     (v_mfma_f32_32x32x16_f16), A = X, B = W^T, so lane l holds output row
//     (l%32) and stores of Y are contiguous along rows;
//   - W is decoded ONCE per workgroup: per K-step of 64 (one Q4_K chunk) waves
//     0..2 each decode one row tile (lane = row l%32, half l/32 of the chunk's
//     32 code bytes, loaded straight from global memory with the superblock
//     header) into four fp16 B fragments and write them to LDS, where all four
//     multiplying waves read them.  Wave 3 runs the same instruction stream on
//     wave 2's rows and stores the same values: no branch in the stream.  The
//     fragments of step ks+1 are decoded between the MFMAs of step ks;
//   - waves 4..7 only move X, with direct global -> LDS loads
//     (global_load_lds_dwordx4: no registers in between), four buffers, two
//     steps in flight.  A direct load places lane l's 16 bytes at base + 16*l,
//     so padding rows is not possible; instead the 16-byte chunk c of token row
//     t is stored at position c ^ (t & 7) (the source address is permuted),
//     which spreads the fragment reads of consecutive rows over all banks;
//   - one barrier per K-step.  It is a bare s_barrier behind counted waits:
//     __syncthreads() carries a workgroup fence for which the compiler waits for
//     every outstanding load, the steps in flight included.
// K order inside a 64-step is permuted consistently on both operands:
// MFMA q (0..3) of chunk c takes, for lane half h, elements
//   q<2 : 64c + 16h + 8q .. +7        (low nibbles of code bytes 8q..8q+7)
//   q>=2: 64c + 32 + 16h + 8(q-2) ..  (high nibbles of the same bytes)
#include "lev_common.hpp"

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kBM = 256;          // tokens per workgroup
constexpr int kSBN = 96;          // rows per workgroup
constexpr int kSRT = 3;           // 32-row tiles per wave
constexpr int kSMT = 2;           // 32-token tiles per wave
constexpr int kKS = 64;           // K-step (one chunk)
constexpr int kXRow = 128;        // bytes per token row in LDS
constexpr int kXBuf = kBM * kXRow;
constexpr int kXBufs = 4;         // X buffers in LDS: the step in use, the next (landed), two in flight
constexpr int kBFrag = 64 * 16;                 // one B fragment: 16 bytes per lane
constexpr int kBBuf = 4 * kSRT * kBFrag;        // [q][row tile][lane], one K-step; two of them
constexpr int kSThreads = 512;                  // four multiplying waves and four that load X

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
    asm("" : "+v"(w32));
    return (_Float16)w32;
}

// 8 weights (one per code byte of the two dwords, nibble selected by `hi`)
// -> fp16 B fragment, bit-exact with fp16(f32(d1*q - mm)).
__device__ __forceinline__ f16x8 q4k_frag(uint32_t q0, uint32_t q1, bool hi, float d1, float mm) {
    uint32_t a = hi ? (q0 >> 4) : q0, b = hi ? (q1 >> 4) : q1;
    a &= 0x0F0F0F0Fu;
    b &= 0x0F0F0F0Fu;
    // opaque from here: the compiler would otherwise fold the mask into four
    // bit-field extracts per dword instead of using v_cvt_f32_ubyte0..3 directly
    asm("" : "+v"(a));
    asm("" : "+v"(b));
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

// s_waitcnt vmcnt(n) leaves at most n loads outstanding; loads complete in
// issue order, so everything older than the n newest has landed.  Encoding:
// vmcnt in bits 3:0 and 15:14, expcnt (6:4) and lgkmcnt (11:8) left at "any".
#define LEV_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 0xF) | (((n) >> 4) << 14) | (7 << 4) | (15 << 8))

// grid (ceil(rows/96), ceil(tokens/256)); LDS kXBufs*kXBuf + 2*kBBuf bytes.
__global__ void __launch_bounds__(kSThreads)
q4_k_gemm_kernel(const uint8_t *__restrict__ w, const uint16_t *__restrict__ x,
                 float *__restrict__ y, uint32_t in_dim, uint32_t rows, uint32_t tokens) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    uint8_t *const ldsb = lds + kXBufs * kXBuf;
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t lr = lane & 31u, lh = lane >> 5;
    const uint32_t row0 = blockIdx.x * kSBN;
    const uint32_t tok0 = blockIdx.y * kBM;
    const uint32_t nsb = in_dim / 256u;
    const uint32_t drt = wave < 3u ? wave : 2u;          // row tile this wave decodes
    const uint32_t drow = row0 + 32u * drt + lr;
    const uint8_t *const wrow = w + (uint64_t)(drow < rows ? drow : rows - 1u) * nsb * 144u;

    const uint32_t nsteps = nsb * 4u;

    // Waves 4..7 only move X, one on each SIMD: per K-step each issues 8 direct
    // global -> LDS loads (eight token rows of 128 bytes per load).  The path from
    // L1 takes 64 bytes a cycle, so the 32 KB of a step keep it busy for most of
    // the step; a wave that multiplies would stall at every request until the path
    // accepts it, these have nothing else to do.  Step ks+2 goes into the buffer
    // step ks-2 used (every wave has passed barrier ks-1, hence finished reading
    // it); vmcnt(8) before barrier ks leaves only the loads of step ks+1
    // outstanding.  Addresses are a uniform base plus a 32-bit lane offset fixed
    // for the whole kernel, so a request costs no vector instruction.
    if (wave >= 4u) {
        const uint32_t lw = __builtin_amdgcn_readfirstlane(wave) - 4u, ltok = lane >> 3, lpos = lane & 7u;
        const uint8_t *const xtile = reinterpret_cast<const uint8_t *>(x) + (uint64_t)tok0 * in_dim * 2u;
        uint32_t voff[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const uint32_t tl = 8u * (8u * lw + j) + ltok;
            const uint32_t t = tok0 + tl < tokens ? tl : tokens - 1u - tok0;
            voff[j] = t * in_dim * 2u + 16u * (lpos ^ (ltok & 7u));
        }
        auto x_request = [&](uint32_t kstep, uint32_t buf) {
            const uint8_t *const xk = xtile + (uint64_t)kstep * (kKS * 2u);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                uint8_t *dst = lds + buf * kXBuf + (8u * lw + j) * 1024u;
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(xk + voff[j]),
                                                 (__attribute__((address_space(3))) void *)dst, 16, 0, 0);
            }
        };
        x_request(0, 0);
        x_request(1 < nsteps ? 1 : nsteps - 1, 1);
        for (uint32_t ks = 0; ks < nsteps; ++ks) {
            LEV_WAIT_VMCNT(8);
            asm volatile("s_barrier" ::: "memory");
            x_request(ks + 2 < nsteps ? ks + 2 : nsteps - 1, (ks + 2) & 3u);
        }
        LEV_WAIT_VMCNT(0);
        return;
    }

    f32x16 acc[kSRT][kSMT];
#pragma unroll
    for (int r = 0; r < kSRT; ++r)
#pragma unroll
        for (int m = 0; m < kSMT; ++m)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[r][m][i] = 0.f;

    // The weights of superblock sb+1 are requested in the first K-step of
    // superblock sb and taken over in its last: with request and first use in one
    // trip of the loop the compiler knows how many loads were issued in between
    // and waits for exactly those (over the loop's back edge it would wait for
    // everything in flight).  Loads are unconditional (clamped at the end) so
    // that no branch forces a wait.
    lev_u32x4 hdr_n, qs_n[4];
    auto w_load = [&](uint32_t sb) {
        const uint32_t sbc = sb < nsb ? sb : nsb - 1u;
        const uint8_t *blk = wrow + (uint64_t)sbc * 144u;
        hdr_n = *reinterpret_cast<const lev_u32x4 *>(blk);
#pragma unroll
        for (int cc = 0; cc < 4; ++cc)
            qs_n[cc] = *reinterpret_cast<const lev_u32x4 *>(blk + 16u + 32u * cc + 16u * lh);
    };
    lev_u32x4 qs[4];
    float d1[8], mm[8];
    auto take = [&]() {
#pragma unroll
        for (int cc = 0; cc < 4; ++cc) {
            qs[cc] = qs_n[cc];
            // touched here so that the wait for these loads sits here and not at their first use
            asm volatile("" : "+v"(qs[cc].x), "+v"(qs[cc].y), "+v"(qs[cc].z), "+v"(qs[cc].w));
        }
        q4k_all_factors(hdr_n, d1, mm);
    };
    w_load(0);
    take();
    {   // chunk 0 of superblock 0 -> B buffer 0
        const lev_u32x4 q = qs[0];
        f16x8 f[4];
        f[0] = q4k_frag(q.x, q.y, false, d1[0], mm[0]);
        f[1] = q4k_frag(q.z, q.w, false, d1[0], mm[0]);
        f[2] = q4k_frag(q.x, q.y, true, d1[1], mm[1]);
        f[3] = q4k_frag(q.z, q.w, true, d1[1], mm[1]);
#pragma unroll
        for (int qq = 0; qq < 4; ++qq)
            *reinterpret_cast<f16x8 *>(ldsb + (qq * kSRT + drt) * kBFrag + lane * 16u) = f[qq];
    }
    // The loop is rotated by two MFMA groups: groups 2 and 3 of a step are
    // multiplied AFTER the barrier of the next step, from fragments read before
    // it, so that the matrix cores have work while the first fragments of the
    // new step come in from LDS (with X landing in LDS at the same time such a
    // read takes several hundred cycles).  A trip is therefore
    //   barrier(ks) | read group 0 | MFMA 2, 3 of ks-1 (reading group 1) |
    //   MFMA 0, 1 of ks (reading groups 2, 3)
    // with fragment p of chunk ks+1 decoded in phase p, so the B fragments of
    // step ks+1 are complete (and the reads of step ks done) before barrier(ks+1).
    // The first trip multiplies zero fragments in its phases 0 and 1.
    f16x8 a_buf[4][kSMT], b_buf[4][kSRT];
#pragma unroll
    for (int g = 2; g < 4; ++g) {
#pragma unroll
        for (int m = 0; m < kSMT; ++m)
#pragma unroll
            for (int i = 0; i < 8; ++i) a_buf[g][m][i] = (_Float16)0.f;
#pragma unroll
        for (int r = 0; r < kSRT; ++r)
#pragma unroll
            for (int i = 0; i < 8; ++i) b_buf[g][r][i] = (_Float16)0.f;
    }
    for (uint32_t sb = 0; sb < nsb; ++sb) {
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const uint32_t ks = sb * 4u + c;
            // this wave's B fragments of step ks have left for LDS and its reads of
            // step ks-1 have arrived (the bare barrier waits for neither); the
            // loader waves have waited for X of step ks
            __builtin_amdgcn_s_waitcnt(0xC07F);   // lgkmcnt(0), vmcnt and expcnt left open
            asm volatile("s_barrier" ::: "memory");

            const int cn = c == 3 ? 0 : c + 1;
            const uint8_t *xb = lds + (ks & 3u) * kXBuf + (wave * 64u + lr) * kXRow;
            const uint8_t *bb = ldsb + (ks & 1u) * kBBuf + lane * 16u;
            uint8_t *bw = ldsb + ((ks + 1u) & 1u) * kBBuf + drt * kBFrag + lane * 16u;
            // fragment `which` (use order a0 b0 b1 b2 a1) of MFMA group qq
            auto frag_read_one = [&](int qq, int which) {
                if (which == 0 || which == 4) {
                    const int m = which == 0 ? 0 : 1;
                    const uint32_t chunk = 2u * lh + (qq < 2 ? qq : 2u + qq);
                    const uint32_t koff = 16u * (chunk ^ (lr & 7u));
                    a_buf[qq][m] = *reinterpret_cast<const f16x8 *>(xb + m * 32 * kXRow + koff);
                } else {
                    const int r = which - 1;
                    b_buf[qq][r] = *reinterpret_cast<const f16x8 *>(bb + (qq * kSRT + r) * kBFrag);
                }
            };
#pragma unroll
            for (int f = 0; f < 5; ++f) frag_read_one(0, f);
            if (c == 0) w_load(sb + 1u);
            if (c == 3) take();
#pragma unroll
            for (int ph = 0; ph < 4; ++ph) {
                const int qq = (ph + 2) & 3;   // the MFMA group of this phase
                const int rg = ph == 0 ? 1 : ph;   // the group read in this phase (none in phase 1)
                // fragment ph of the NEXT chunk is decoded behind this phase's MFMAs
                const lev_u32x4 w4 = qs[cn];
                uint32_t c0 = (ph & 1) ? w4.z : w4.x, c1 = (ph & 1) ? w4.w : w4.y;
                if (ph >= 2) {
                    c0 >>= 4;
                    c1 >>= 4;
                }
                c0 &= 0x0F0F0F0Fu;
                c1 &= 0x0F0F0F0Fu;
                asm("" : "+v"(c0));
                asm("" : "+v"(c1));
                const float fd = d1[2 * cn + (ph >> 1)], fm = mm[2 * cn + (ph >> 1)];
                f16x8 nf;
                // Six slots of { one MFMA, a few other instructions }: a wave issues in
                // order and an MFMA holds the matrix pipe for 32 cycles, so what is
                // issued behind it within that time is free.  Five slots take one
                // fragment read (two groups ahead of its use), four take two weights
                // of the decode.
#pragma unroll
                for (int i = 0; i < 6; ++i) {
                    const int r = i % 3, m = i / 3;
                    acc[r][m] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a_buf[qq][m], b_buf[qq][r], acc[r][m], 0, 0, 0);
                    if (ph != 1 && i < 5) frag_read_one(rg, i);
                    if (r != 2) {
                        const int s4 = 2 * m + r;
                        const uint32_t cw = s4 < 2 ? c0 : c1;
                        const float e0 = (s4 & 1) ? (float)((cw >> 16) & 0xFFu) : (float)(cw & 0xFFu);
                        const float e1 = (s4 & 1) ? (float)(cw >> 24) : (float)((cw >> 8) & 0xFFu);
                        nf[2 * s4] = q4k_weight_f16(fd, e0, fm);
                        nf[2 * s4 + 1] = q4k_weight_f16(fd, e1, fm);
                    }
                    // wave 3 decoded wave 2's rows: it stores the same values to the same place,
                    // which keeps the stream free of branches (a branch makes the compiler wait
                    // for every LDS operation at the join)
                    if (i == 5) *reinterpret_cast<f16x8 *>(bw + ph * kSRT * kBFrag) = nf;
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
    }
    // groups 2 and 3 of the last step
#pragma unroll
    for (int g = 2; g < 4; ++g)
#pragma unroll
        for (int i = 0; i < 6; ++i) {
            const int r = i % 3, m = i / 3;
            acc[r][m] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a_buf[g][m], b_buf[g][r], acc[r][m], 0, 0, 0);
        }

#pragma unroll
    for (int r = 0; r < kSRT; ++r) {
        const uint32_t my_row = row0 + 32u * r + lr;
        if (my_row >= rows) continue;
#pragma unroll
        for (int m = 0; m < kSMT; ++m)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                uint32_t t = tok0 + wave * 64u + m * 32 + 8 * (i / 4) + 4 * lh + (i % 4);
                if (t < tokens) y[(uint64_t)t * rows + my_row] = acc[r][m][i];
            }
    }
}


}  // namespace

hipError_t lev_q4_k_gemm_launch(lev_ctx *ctx, const uint8_t *w, const uint16_t *x, float *y,
                                uint32_t in_dim, uint32_t rows, uint32_t tokens) {
    static bool attr_set = false;
    const size_t lds = (size_t)kXBufs * kXBuf + 2 * kBBuf;
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&q4_k_gemm_kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    dim3 grid((rows + kSBN - 1) / kSBN, (tokens + kBM - 1) / kBM);
    hipLaunchKernelGGL(q4_k_gemm_kernel, grid, dim3(kSThreads), lds, ctx->stream, w, x, y, in_dim,
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
    if (in_dim > (1u << 22))   // the X loaders keep 32-bit byte offsets inside a 256-token tile
        return lev_fail(ctx, LEV_ERR_BAD_DIMENSIONS, "q4_k_gemm_prefill: in_dim %u above 4194304", in_dim);
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

// Routed Q4_0 experts for MANY tokens on gfx950: (token, slot) pairs are
// grouped by expert, and each expert's weights are streamed once and applied
// to all of its tokens on the matrix cores.
//
// Stands in for runMoeBatchedRouted applied token after token
// (Sources/LeviathanCore/Gemma4.swift:2073, per-slot loop :3856-3880;
// moegen_gu/act/dn, MoELowering.swift:749-835): same results per pair, same
// slot-ordered f32 merge; only the order in which pairs are visited changes.
// With one launch per (token, slot) every pair streams its expert's 2.65 MB
// again (64 tokens x top-8 = 512 x 2.65 MB against 126 distinct experts).
//
// Pipeline (all on the context's stream):
//   1. group:  histogram of expert ids -> offsets; list of pairs per expert;
//              beside it, one workgroup per token writes x as two fp16 planes
//              (high + low half, after a power-of-two row scale), in the k-slot
//              order of step 2.
//   2. gate/up on MFMA -> act = gelu_tanh(g)*u (f32, [pair][inter]) and the
//              largest |act| of every pair (atomic maximum on the bit patterns).
//   3. down on MFMA -> dn (f32, [pair][hidden]); it splits act into planes
//              while it copies the rows into LDS.
//   4. merge:  y[t] = sum over slots, IN SLOT ORDER, fmaf(w_slot, dn_slot, acc).
//
// MFMA formulation (v_mfma_f32_16x16x32_f16), per Q4_0 block of 32 weights:
//   B = 16 weight rows x the block's 32 codes as exact fp16 integers n-8
//       (mask, OR in 1024's exponent, subtract 1032: two instructions per two
//       weights, no conversion);
//   A = up to 8 tokens' activations of that block, fp16 high and low halves
//       (two MFMAs), x = hi + lo to 2^-22;
//   the output lane of weight row n is the lane that holds row n's block scale
//   d, so y += d * (A.B) needs no exchange.
// A wave fetches the 144 bytes of eight blocks of each of its 16 rows as they lie
// in memory, 16 bytes per lane with consecutive lanes on consecutive bytes of a row
// (the L1 looks a 32-byte sector up once per four lanes that touch it: lanes on
// different rows cost a lookup each, and with a block pair per lane the lookups,
// not the bytes, kept the L1 busy for more than half of the kernel), parks them in
// a small wave-private LDS area, and every lane reads from there the four code
// bytes (both nibbles: eight weights) and the scale it multiplies.
#include "moe_grouped.hpp"

#include <cstdlib>

namespace {

constexpr int kGrpThreads = 1024;
constexpr int kGrpWaves = kGrpThreads / LEV_WAVE;
constexpr int kNC = 12;                // token columns per pass (of the 16 an MFMA takes; the planes of 16 would not
                                       // fit the LDS at hidden 2048).  An expert with more pairs takes another pass over
                                       // its weights, and its workgroups that much longer than all the others: at 64
                                       // tokens x top-8 over 128 experts one in fifty has more than 8 pairs (a layer then
                                       // measured 172 us instead of 122), one in three thousand more than 12
constexpr int kFlagBadExpertId = 1;    // same bit as the per-token kernels
constexpr uint32_t kGrpRowBytes = 152;        // a row of a wave's area: the 144 bytes of eight blocks + 8: 38 dwords,
                                              // so that the 16 rows start in 16 different even banks of the 32
constexpr uint32_t kGrpRawBytes = 16 * kGrpRowBytes;
constexpr int kGrpLoads = 3;                  // 16-byte loads per lane and group: 16 rows x 144 bytes over 64 lanes
constexpr size_t kGrpStaticLds = (size_t)2 * (kGrpWaves / 2) * 16 * kNC * 4 + 1024;   // gate values, pair records

typedef _Float16 g_h8 __attribute__((ext_vector_type(8)));
typedef uint32_t g_u4 __attribute__((ext_vector_type(4)));
typedef uint32_t g_u2 __attribute__((ext_vector_type(2)));

// ---------------------------------------------------------------------------
// Activation planes.  A row is scaled by the power of two that brings its maximum into [1, 2)
// (zero, denormal and non-finite maxima: no scaling) and split into fp16 high and low halves;
// run 4b + g of a row holds elements 4g, 4g+2, 4g+1, 4g+3, then 16+4g, 16+4g+2, 16+4g+1, 16+4g+3 of
// block b: the weights in code bytes 4g..4g+3 of the block (low nibbles, then high nibbles), in the
// order in which the masks of the matrix-core kernel deliver them.
// ---------------------------------------------------------------------------
struct grp_scale { float scale, unscale; };
__device__ __forceinline__ grp_scale grp_row_scale(uint32_t max_bits) {
    uint32_t ex = (max_bits >> 23) & 0xFFu;
    if (ex == 0u || ex >= 254u) ex = 127u;
    return grp_scale{__uint_as_float((254u - ex) << 23), __uint_as_float(ex << 23)};
}
__device__ __forceinline__ void grp_split_run(lev_f32x4 a, lev_f32x4 b, float scale, g_h8 &h, g_h8 &l) {
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
    a = a * scale;
    b = b * scale;
    const float m[8] = {a.x, a.z, a.y, a.w, b.x, b.z, b.y, b.w};
#pragma unroll
    for (int k = 0; k < 8; k += 2) {
        const f32x2 pair = {m[k], m[k + 1]};
        const f16x2 hp = __builtin_convertvector(pair, f16x2);
        const f32x2 rest = {pair.x - (float)hp.x, pair.y - (float)hp.y};
        const f16x2 lp = __builtin_convertvector(rest, f16x2);
        h[k] = hp.x; h[k + 1] = hp.y;
        l[k] = lp.x; l[k + 1] = lp.y;
    }
}

// ---------------------------------------------------------------------------
// 1. group pairs by expert.  One workgroup.  A pair is dropped (and flagged)
// when its id is out of range or repeats an earlier slot of the same token,
// as MoEModelBinding.offsets requires (MoEModelBinding.swift:174-214).
// goff[e] .. goff[e+1]: expert e's pairs in glist; valid[p]: pair p takes part.
// ---------------------------------------------------------------------------
// Workgroups 1..tokens: the fp16 planes of x[t][:] and its row maximum (bit pattern of the largest
// |x|; NaNs are passed over, as fmaxf does).  Workgroup 0 also clears amax (the per-pair maxima
// step 2 builds).
__global__ void __launch_bounds__(1024)
moe_group_kernel(const int32_t *__restrict__ ids, uint32_t pairs, uint32_t experts, uint32_t top_k,
                 int32_t *__restrict__ goff, int32_t *__restrict__ glist,
                 uint8_t *__restrict__ valid, int *__restrict__ flag, const float *__restrict__ x,
                 uint32_t hidden, _Float16 *__restrict__ xh, _Float16 *__restrict__ xl,
                 uint32_t *__restrict__ xmax, uint32_t *__restrict__ amax) {
    extern __shared__ int32_t s_cnt[];          // [experts] counts, then [experts] cursors
    int32_t *s_cur = s_cnt + experts;
    const uint32_t tid = threadIdx.x;
    if (blockIdx.x != 0u) {
        __shared__ float s_max[16];
        const uint32_t t = blockIdx.x - 1u, runs = hidden >> 3;
        const lev_f32x4 *s4 = reinterpret_cast<const lev_f32x4 *>(x + (uint64_t)t * hidden);
        float mx = 0.f;
        for (uint32_t q = tid; q < 2u * runs; q += 1024u) {
            const lev_f32x4 v = s4[q];
            mx = fmaxf(mx, fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
        if ((tid & 63u) == 0u) s_max[tid >> 6] = mx;
        __syncthreads();
        float m = s_max[0];
        for (int w = 1; w < 16; ++w) m = fmaxf(m, s_max[w]);
        if (tid == 0) xmax[t] = __float_as_uint(m);
        const float scale = grp_row_scale(__float_as_uint(m)).scale;
        for (uint32_t q = tid; q < runs; q += 1024u) {
            g_h8 h, l;
            grp_split_run(s4[8u * (q >> 2) + (q & 3u)], s4[8u * (q >> 2) + 4u + (q & 3u)], scale, h, l);
            *reinterpret_cast<g_h8 *>(xh + (uint64_t)t * hidden + 8u * q) = h;
            *reinterpret_cast<g_h8 *>(xl + (uint64_t)t * hidden + 8u * q) = l;
        }
        return;
    }
    for (uint32_t p = tid; p < pairs; p += 1024u) amax[p] = 0u;
    for (uint32_t e = tid; e < experts; e += 1024u) s_cnt[e] = 0;
    __syncthreads();
    bool bad_seen = false;
    for (uint32_t p = tid; p < pairs; p += 1024u) {
        const int32_t e = ids[p];
        bool ok = e >= 0 && (uint32_t)e < experts;
        const uint32_t slot = p % top_k, first = p - slot;
        for (uint32_t k = 0; k < top_k && ok; ++k)
            if (k != slot && ids[first + k] == e) ok = false;   // both copies of a duplicate are dropped
        valid[p] = ok ? 1 : 0;
        if (ok) atomicAdd(&s_cnt[e], 1);
        bad_seen = bad_seen || !ok;
    }
    if (bad_seen) atomicOr(flag, kFlagBadExpertId);
    __syncthreads();
    // exclusive scan of the counts (experts <= 4096): thread i takes experts 4i..4i+3, the waves scan
    // their threads' sums by shuffles and meet in LDS
    {
        __shared__ int32_t s_wave[16];
        int32_t c4[4], local = 0;
#pragma unroll
        for (uint32_t k = 0; k < 4u; ++k) {
            const uint32_t e = 4u * tid + k;
            c4[k] = e < experts ? s_cnt[e] : 0;
            local += c4[k];
        }
        int32_t incl = local;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int32_t o = __shfl_up(incl, off);
            if ((int)(tid & 63u) >= off) incl += o;
        }
        if ((tid & 63u) == 63u) s_wave[tid >> 6] = incl;
        __syncthreads();
        int32_t run = incl - local;
        for (uint32_t w = 0; w < (tid >> 6); ++w) run += s_wave[w];
#pragma unroll
        for (uint32_t k = 0; k < 4u; ++k) {
            const uint32_t e = 4u * tid + k;
            if (e <= experts) goff[e] = run;
            if (e < experts) s_cur[e] = run;
            run += c4[k];
        }
        // 4096 experts: the total has no thread of its own (thread i owns 4i..4i+3 <= 4095)
        if (4u * tid + 4u == experts && experts == 4096u) goff[experts] = run;
    }
    __syncthreads();
    // The order of an expert's pairs in the list depends on the atomics; no
    // result does: every pair is computed independently and owns its outputs.
    for (uint32_t p = tid; p < pairs; p += 1024u)
        if (valid[p]) glist[atomicAdd(&s_cur[ids[p]], 1)] = (int32_t)p;
}

// ---------------------------------------------------------------------------
// 2./3. grouped matrix-core kernel, 16 waves.  Down: grid (row tiles of 256,
// experts), wave w owns rows 16w..16w+15 of the tile.  PAIRED (gate/up): grid
// (row tiles of 128, experts), waves 0..7 own the tile's gate rows, waves 8..15
// the same rows of the up matrix; gate values meet the up waves in LDS.
// Column j of a pass is pair glist[goff[e] + pass*8 + j]; its activation row is
// the pair's token (PAIRED: gate/up read x) or the pair itself (down reads act).
// ---------------------------------------------------------------------------

// the 4 code bytes a lane takes of one block -> B operand: fp16 integers n - 8, low nibbles
// of bytes (0, 2), (1, 3), then the high nibbles; mask and magic arrive in registers so that
// (v & mask) | magic is ONE v_and_or_b32.
__device__ __forceinline__ g_h8 q4_0_operand(uint32_t codes, uint32_t mask, uint32_t magic) {
    typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
    const f16x2 bias = {(_Float16)1032.0f, (_Float16)1032.0f};
    auto two = [&](uint32_t v) {
        // 0x6400 | n is the fp16 number 1024 + n
        const f16x2 h = __builtin_bit_cast(f16x2, (v & mask) | magic);
        return __builtin_bit_cast(uint32_t, h - bias);
    };
    g_u4 bits;
    bits.x = two(codes);
    bits.y = two(codes >> 8);
    bits.z = two(codes >> 4);
    bits.w = two(codes >> 12);
    return __builtin_bit_cast(g_h8, bits);
}

template <bool PAIRED>
__global__ void __launch_bounds__(kGrpThreads)
moe_grouped_kernel(lev_moe_grouped_args a, uint32_t tiles_per_wg, const float *__restrict__ src,
                   const _Float16 *__restrict__ src_h, const _Float16 *__restrict__ src_l,
                   const uint32_t *__restrict__ src_max, const int32_t *__restrict__ goff,
                   const int32_t *__restrict__ glist, float *__restrict__ out,
                   uint32_t *__restrict__ out_max) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const uint32_t in_len = PAIRED ? a.hidden : a.inter;
    const uint32_t out_rows = PAIRED ? a.inter : a.hidden;
    const uint32_t nblk = in_len >> 5, runs = in_len >> 3;
    const uint32_t e = blockIdx.y;
    const int32_t first = goff[e];
    const uint32_t n = (uint32_t)(goff[e + 1] - first);
    if (n == 0u) return;

    const uint32_t plane = runs * kNC * 8u;                      // halfs
    _Float16 *sxh = reinterpret_cast<_Float16 *>(smem);           // [run][col][8]
    _Float16 *sxl = sxh + plane;
    // wave-private area: the 144 bytes of a group of eight blocks of each of the wave's 16 rows (+ 8 of padding)
    uint8_t *xch = reinterpret_cast<uint8_t *>(sxl + plane);
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    uint8_t *area = xch + wave * kGrpRawBytes;
    __shared__ int32_t s_pair[kNC];
    __shared__ float s_us[kNC], s_scale[kNC];
    __shared__ float s_gate[PAIRED ? 2 * (kGrpWaves / 2) * 16 * kNC : 1];   // [tile parity][tile row][col]

    const uint32_t r = lane & 15u, g = lane >> 4;
    const uint32_t is_up = PAIRED ? wave / (kGrpWaves / 2) : 0u;
    const uint32_t wv = PAIRED ? wave % (kGrpWaves / 2) : wave;          // 16-row slice of a tile
    const uint32_t tile_rows = PAIRED ? (kGrpWaves / 2) * 16 : kGrpWaves * 16;
    const uint32_t ntile = (out_rows + tile_rows - 1u) / tile_rows;
    // this workgroup's row tiles: the activation planes are staged once for all of them and the
    // weight requests run ahead across tile boundaries
    const uint32_t t0 = blockIdx.x * tiles_per_wg;
    const uint32_t t1 = t0 + tiles_per_wg < ntile ? t0 + tiles_per_wg : ntile;
    const uint64_t row_bytes = (uint64_t)nblk * 18u;
    const uint8_t *mat;
    if (PAIRED)
        mat = a.base + (is_up ? a.up_off + e * a.up_stride : a.gate_off + e * a.gate_stride);
    else
        mat = a.base + a.down_off + e * a.down_stride;

    // groups of 8 blocks = 144 bytes = nine 16-byte pieces per row; lane l fetches pieces l, l + 64
    // and (lanes 0..15; the others repeat the last one) l + 128 of the 144 of a group, piece q being
    // piece q % 9 of row q / 9, and parks it in that row of the wave's area (8-byte aligned: two
    // halves; five 8-byte loads per lane instead measured 6 % slower)
    const uint32_t ngrp = nblk >> 3;
    uint32_t prow[kGrpLoads], poff[kGrpLoads], pdst[kGrpLoads];
#pragma unroll
    for (int j = 0; j < kGrpLoads; ++j) {
        const uint32_t q = lane + 64u * j < 143u ? lane + 64u * j : 143u;
        prow[j] = q / 9u;
        poff[j] = (q % 9u) * 16u;
        pdst[j] = prow[j] * kGrpRowBytes + poff[j];
    }
    auto fetch = [&](uint32_t tile, uint32_t grp, g_u4 (&D)[kGrpLoads]) {
        const uint32_t tc = tile < t1 ? tile : t1 - 1u;          // past the end: any valid address
        const uint32_t row0 = tc * tile_rows + wv * 16u;
#pragma unroll
        for (int j = 0; j < kGrpLoads; ++j) {
            const uint32_t row = row0 + prow[j];
            const uint32_t rowc = row < out_rows ? row : out_rows - 1u;
            const lev_u32x4_a4 v =
                *reinterpret_cast<const lev_u32x4_a4 *>(mat + rowc * row_bytes + (uint64_t)grp * 144u + poff[j]);
            D[j] = g_u4{v.v[0], v.v[1], v.v[2], v.v[3]};
        }
    };
    uint32_t k_mask = 0x000F000Fu, k_magic = 0x64006400u;
    asm("" : "+v"(k_mask), "+v"(k_magic));   // keep both in registers (see q4_0_operand)
    const uint8_t *const my_row = area + r * kGrpRowBytes;    // this lane's weight row in the area
    const uint32_t colc = r < (uint32_t)kNC ? r : (uint32_t)kNC - 1u;   // A rows past kNC: any valid address

    for (uint32_t pass = 0; pass * kNC < n; ++pass) {
        const uint32_t ncols = n - pass * kNC < (uint32_t)kNC ? n - pass * kNC : (uint32_t)kNC;
        // the first weights are requested ahead of everything that only concerns the activations
        g_u4 Dc[kGrpLoads], Dn[kGrpLoads];
        uint32_t ft = t0, fg = 0;                                 // the next group to request
        auto advance = [&] { if (++fg == ngrp) { fg = 0; ++ft; } };
        fetch(ft, fg, Dc);
        advance();
        __syncthreads();   // previous pass done with the planes and s_pair
        if (tid < (uint32_t)kNC) {
            // columns past the end repeat the last pair (never stored)
            const int32_t p = glist[first + pass * kNC + (tid < ncols ? tid : ncols - 1u)];
            s_pair[tid] = p;
            const grp_scale sc = grp_row_scale(src_max[PAIRED ? p / (int32_t)a.top_k : p]);
            s_us[tid] = sc.unscale;
            s_scale[tid] = sc.scale;
        }
        __syncthreads();
        // stage the pass's columns in runs of 8 values -> 16 bytes per plane.  Consecutive threads take the kNC columns of one
        // run, then the next run: their LDS writes are contiguous (column-major threads wrote
        // 16 bytes at a stride of kNC*16 bytes, every lane of a wave into the same four
        // banks).  Columns past the end keep what the area held: an MFMA row of A only reaches its
        // own row of outputs, which is never stored.
        for (uint32_t i = tid; i < runs * kNC; i += kGrpThreads) {
            const uint32_t c = i % kNC, q = i / kNC;
            if (c < ncols) {
                const int32_t p = s_pair[c];
                g_h8 h, l;
                if (PAIRED) {
                    // x: planes written beside the grouping
                    const uint64_t at = (uint64_t)(p / (int32_t)a.top_k) * in_len + 8u * q;
                    h = *reinterpret_cast<const g_h8 *>(src_h + at);
                    l = *reinterpret_cast<const g_h8 *>(src_l + at);
                } else {
                    // act: split here, its row maximum was only complete when gate/up ended
                    const lev_f32x4 *s4 = reinterpret_cast<const lev_f32x4 *>(src + (uint64_t)p * in_len);
                    grp_split_run(s4[8u * (q >> 2) + (q & 3u)], s4[8u * (q >> 2) + 4u + (q & 3u)], s_scale[c], h, l);
                }
                *reinterpret_cast<g_h8 *>(sxh + (q * kNC + c) * 8u) = h;
                *reinterpret_cast<g_h8 *>(sxl + (q * kNC + c) * 8u) = l;
            }
        }
        __syncthreads();

        uint32_t cmax[4] = {0u, 0u, 0u, 0u};
        for (uint32_t tile = t0; tile < t1; ++tile) {
            lev_f32x4 y = {0.f, 0.f, 0.f, 0.f};
            for (uint32_t grp = 0; grp < ngrp; ++grp) {
                // the next group (of this tile or the next) is requested before this one is multiplied
                // (two groups on their way measured 3-6 % slower, before and after the loads were made to follow the rows);
                // unconditional (clamped past the end): no branch around loads
                fetch(ft, fg, Dn);
                advance();
                // park the group as it lies in memory
#pragma unroll
                for (int j = 0; j < kGrpLoads; ++j) {
                    *reinterpret_cast<g_u2 *>(area + pdst[j]) = g_u2{Dc[j].x, Dc[j].y};
                    *reinterpret_cast<g_u2 *>(area + pdst[j] + 8u) = g_u2{Dc[j].z, Dc[j].w};
                }
                // wave-private area: the hardware runs one wave's LDS accesses in order
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
                for (uint32_t b = 0; b < 8u; ++b) {
                    const uint32_t at = (((grp * 8u + b) * 4u + g) * kNC + colc) * 8u;
                    const g_h8 Ah = *reinterpret_cast<const g_h8 *>(sxh + at);
                    const g_h8 Al = *reinterpret_cast<const g_h8 *>(sxl + at);
                    // code bytes 4g..4g+3 of block b start at byte 18 b + 2 + 4 g of the row's 144: on a
                    // dword boundary for odd b, two bytes behind one for even b
                    uint32_t codes;
                    if (b & 1u) {
                        codes = *reinterpret_cast<const uint32_t *>(my_row + 18u * b + 2u + 4u * g);
                    } else {
                        const lev_u32x2_a4 two_dw = *reinterpret_cast<const lev_u32x2_a4 *>(my_row + 18u * b + 4u * g);
                        codes = __builtin_amdgcn_alignbit(two_dw.v[1], two_dw.v[0], 16);
                    }
                    const _Float16 d = *reinterpret_cast<const _Float16 *>(my_row + 18u * b);
                    const g_h8 B = q4_0_operand(codes, k_mask, k_magic);
                    lev_f32x4 acc = {0.f, 0.f, 0.f, 0.f};
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(Ah, B, acc, 0, 0, 0);
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(Al, B, acc, 0, 0, 0);
#pragma unroll
                    for (int i = 0; i < 4; ++i) y[i] = fmaf((float)d, acc[i], y[i]);
                }
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();   // reads done before the next group's writes
#pragma unroll
                for (int k = 0; k < kGrpLoads; ++k) Dc[k] = Dn[k];
            }

            // output lane (r, g): weight row r of the tile, columns 4g..4g+3
            const uint32_t row = tile * tile_rows + wv * 16u + r;
            // gate values wait for the up waves in the buffer of the tile's parity: a gate wave
            // cannot reach the same buffer again before the up waves have passed the barrier of
            // the tile between, which lies behind their reads
            float *sg = s_gate + (PAIRED ? ((tile - t0) & 1u) * ((kGrpWaves / 2) * 16 * kNC) : 0u);
            if (PAIRED) {
                if (!is_up) {
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        if (4u * g + i < (uint32_t)kNC) sg[(wv * 16u + r) * kNC + 4u * g + i] = y[i] * s_us[4u * g + i];
                }
                __syncthreads();
            }
            if (!PAIRED || is_up) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const uint32_t col = 4u * g + i;
                    const bool live = col < ncols && row < out_rows;
                    const int32_t p = s_pair[col < (uint32_t)kNC ? col : 0u];
                    float v = 0.f;
                    if (live) {
                        v = y[i] * s_us[col];
                        if (PAIRED) v = lev_gelu_up_value(sg[(wv * 16u + r) * kNC + col], v);
                        out[(uint64_t)p * out_rows + row] = v;
                    }
                    if (PAIRED) {
                        // running maximum of |act| per column over this wave's tiles: the bit patterns
                        // of non-negative floats order as the floats do, and a NaN ranks above every
                        // number (the down stage then leaves the row unscaled)
                        const uint32_t m = __float_as_uint(fabsf(v));
                        cmax[i] = m > cmax[i] ? m : cmax[i];
                    }
                }
            }
        }
        if (PAIRED && is_up) {
            // largest |act| of each of the pass's pairs: over the wave's 16 rows by DPP, then one
            // atomic per column and wave
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                uint32_t m = cmax[i];
#define LEV_GRP_MAXSTEP(CTRL)                                                                          \
                {                                                                                      \
                    const uint32_t o = (uint32_t)__builtin_amdgcn_update_dpp((int)m, (int)m, CTRL, 0xF, 0xF, false); \
                    m = o > m ? o : m;                                                                 \
                }
                LEV_GRP_MAXSTEP(0xB1);    // quad_perm [1,0,3,2]
                LEV_GRP_MAXSTEP(0x4E);    // quad_perm [2,3,0,1]
                LEV_GRP_MAXSTEP(0x141);   // row_half_mirror
                LEV_GRP_MAXSTEP(0x140);   // row_mirror
#undef LEV_GRP_MAXSTEP
                const uint32_t col = 4u * g + (uint32_t)i;
                if (r == 0u && col < ncols && m != 0u) atomicMax(out_max + s_pair[col], m);
            }
        }
    }
}

// 4. merge in slot order (g4_axpy chain, Gemma4.swift:2171-2175); dropped pairs add nothing.
// grid (ceil(hidden / 1024), tokens), 256 threads, four outputs a thread.  Eight slots' rows are
// requested together (a row of a dropped pair was never written: it is read all the same, so that
// no load waits behind a branch, and replaced by zeros), the multiply-adds follow in slot order.
__global__ void __launch_bounds__(256)
moe_merge_kernel(const float *__restrict__ dn, const float *__restrict__ weights,
                 const uint8_t *__restrict__ valid, float *__restrict__ y, uint32_t hidden,
                 uint32_t top_k) {
    const uint32_t t = blockIdx.y, h = (blockIdx.x * 256u + threadIdx.x) * 4u;
    if (h >= hidden) return;
    const bool whole = h + 4u <= hidden && (hidden & 3u) == 0u;   // (hidden is a multiple of 256 on this path)
    lev_f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    for (uint32_t k0 = 0; k0 < top_k; k0 += 8u) {
        lev_f32x4 v[8];
        float w[8];
        bool ok[8];
#pragma unroll
        for (uint32_t u = 0; u < 8u; ++u) {
            const uint32_t p = t * top_k + (k0 + u < top_k ? k0 + u : top_k - 1u);
            const float *row = dn + (uint64_t)p * hidden + h;
            if (whole) {
                v[u] = *reinterpret_cast<const lev_f32x4 *>(row);
            } else {
#pragma unroll
                for (uint32_t c = 0; c < 4u; ++c) v[u][c] = h + c < hidden ? row[c] : 0.f;
            }
            w[u] = weights[p];
            ok[u] = valid[p] != 0 && k0 + u < top_k;
        }
#pragma unroll
        for (uint32_t u = 0; u < 8u; ++u) {
            if (k0 + u >= top_k) break;
            const lev_f32x4 vu = ok[u] ? v[u] : lev_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (uint32_t c = 0; c < 4u; ++c) acc[c] = fmaf(w[u], vu[c], acc[c]);
        }
    }
    if (whole) {
        *reinterpret_cast<lev_f32x4 *>(y + (uint64_t)t * hidden + h) = acc;
    } else {
        for (uint32_t c = 0; c < 4u && h + c < hidden; ++c) y[(uint64_t)t * hidden + h + c] = acc[c];
    }
}

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

struct grouped_layout {
    size_t goff, glist, valid, xh, xl, xmax, amax, dn, total;
};

grouped_layout layout_of(const lev_moe_grouped_args &a) {
    const size_t pairs = (size_t)a.tokens * a.top_k;
    grouped_layout L;
    size_t o = 0;
    L.goff = o; o += align256((a.experts + 1) * 4);
    L.glist = o; o += align256(pairs * 4);
    L.valid = o; o += align256(pairs);
    L.xh = o; o += align256((size_t)a.tokens * a.hidden * 2);
    L.xl = o; o += align256((size_t)a.tokens * a.hidden * 2);
    L.xmax = o; o += align256((size_t)a.tokens * 4);
    L.amax = o; o += align256(pairs * 4);
    L.dn = o; o += align256(pairs * a.hidden * 4);
    L.total = o;
    return L;
}

size_t grouped_lds(uint32_t in_len, bool paired) {
    (void)paired;
    return (size_t)2 * (in_len / 8) * kNC * 16 + (size_t)kGrpWaves * kGrpRawBytes;
}

// Row tiles per workgroup.  A workgroup pays for its activation planes (a chain of dependent reads
// and three barriers) whatever it multiplies afterwards, and its weight requests only run ahead
// inside its own tiles: as many tiles as still leave one workgroup per CU.  The experts that
// take part are not known on the host; at most min(experts, pairs) do.
uint32_t tiles_per_wg(const lev_ctx *ctx, const lev_moe_grouped_args &a, uint32_t tiles, int down) {
    static const char *env[2] = {getenv("LEV_MOE_GROUPED_TILES_GU"), getenv("LEV_MOE_GROUPED_TILES_DN")};
    if (env[down] && atoi(env[down]) > 0) return (uint32_t)atoi(env[down]);
    const uint64_t pairs = (uint64_t)a.tokens * a.top_k;
    const uint64_t active = pairs < a.experts ? pairs : a.experts;
    const uint64_t cus = (uint64_t)ctx->props.multiProcessorCount;
    uint64_t t = (uint64_t)tiles * active / (cus ? cus : 1);
    if (t < 1) t = 1;
    if (t > tiles) t = tiles;
    return (uint32_t)t;
}

}  // namespace

size_t lev_moe_grouped_scratch_bytes(const lev_moe_grouped_args &a) { return layout_of(a).total; }

// Geometry the grouped path serves (the caller also checks 4-byte aligned pools).
bool lev_moe_grouped_usable(const lev_ctx *ctx, const lev_moe_grouped_args &a) {
    const size_t limit = ctx->props.sharedMemPerBlockOptin > ctx->props.sharedMemPerBlock
                             ? ctx->props.sharedMemPerBlockOptin
                             : ctx->props.sharedMemPerBlock;
    return a.hidden % 256u == 0u && a.inter % 256u == 0u && a.experts <= 4096u &&
           (uint64_t)a.tokens * a.top_k <= (1u << 20) && grouped_lds(a.hidden, true) + kGrpStaticLds <= limit &&
           grouped_lds(a.inter, false) + kGrpStaticLds <= limit;
}

// act: f32 [tokens*top_k][inter] (written here, read by the down stage).
hipError_t lev_moe_grouped_launch(lev_ctx *ctx, const lev_moe_grouped_args &a, const float *x,
                                  const int32_t *ids, const float *weights, float *y, float *act,
                                  void *scratch) {
    const grouped_layout L = layout_of(a);
    char *s = static_cast<char *>(scratch);
    int32_t *goff = reinterpret_cast<int32_t *>(s + L.goff);
    int32_t *glist = reinterpret_cast<int32_t *>(s + L.glist);
    uint8_t *valid = reinterpret_cast<uint8_t *>(s + L.valid);
    _Float16 *xh = reinterpret_cast<_Float16 *>(s + L.xh), *xl = reinterpret_cast<_Float16 *>(s + L.xl);
    uint32_t *xmax = reinterpret_cast<uint32_t *>(s + L.xmax), *amax = reinterpret_cast<uint32_t *>(s + L.amax);
    float *dn = reinterpret_cast<float *>(s + L.dn);
    const uint32_t pairs = a.tokens * a.top_k;
    hipError_t e;

    hipLaunchKernelGGL(moe_group_kernel, dim3(1 + a.tokens), dim3(1024), (size_t)2 * a.experts * 4,
                       ctx->stream, ids, pairs, a.experts, a.top_k, goff, glist, valid, ctx->d_flag, x,
                       a.hidden, xh, xl, xmax, amax);
    if ((e = hipGetLastError()) != hipSuccess) return e;

    static size_t lds_set[2] = {0, 0};
    const size_t lds_gu = grouped_lds(a.hidden, true), lds_dn = grouped_lds(a.inter, false);
    if (lds_gu > 48 * 1024 && lds_gu > lds_set[0]) {
        e = hipFuncSetAttribute(reinterpret_cast<const void *>(&moe_grouped_kernel<true>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_gu);
        if (e != hipSuccess) return e;
        lds_set[0] = lds_gu;
    }
    if (lds_dn > 48 * 1024 && lds_dn > lds_set[1]) {
        e = hipFuncSetAttribute(reinterpret_cast<const void *>(&moe_grouped_kernel<false>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_dn);
        if (e != hipSuccess) return e;
        lds_set[1] = lds_dn;
    }
    const uint32_t rows_per_wg = kGrpWaves * 16, rows_per_wg_gu = rows_per_wg / 2;
    const uint32_t tiles_gu = (a.inter + rows_per_wg_gu - 1) / rows_per_wg_gu;
    const uint32_t tiles_dn = (a.hidden + rows_per_wg - 1) / rows_per_wg;
    const uint32_t tpw_gu = tiles_per_wg(ctx, a, tiles_gu, 0), tpw_dn = tiles_per_wg(ctx, a, tiles_dn, 1);
    hipLaunchKernelGGL((moe_grouped_kernel<true>), dim3((tiles_gu + tpw_gu - 1) / tpw_gu, a.experts),
                       dim3(kGrpThreads), lds_gu, ctx->stream, a, tpw_gu, nullptr, xh, xl, xmax, goff, glist, act, amax);
    if ((e = hipGetLastError()) != hipSuccess) return e;
    // rows of act that belong to dropped pairs are never written and never read
    hipLaunchKernelGGL((moe_grouped_kernel<false>), dim3((tiles_dn + tpw_dn - 1) / tpw_dn, a.experts),
                       dim3(kGrpThreads), lds_dn, ctx->stream, a, tpw_dn, act, nullptr, nullptr, amax, goff, glist, dn, nullptr);
    if ((e = hipGetLastError()) != hipSuccess) return e;
    hipLaunchKernelGGL(moe_merge_kernel, dim3((a.hidden + 1023) / 1024, a.tokens), dim3(256), 0, ctx->stream,
                       dn, weights, valid, y, a.hidden, a.top_k);
    return hipGetLastError();
}

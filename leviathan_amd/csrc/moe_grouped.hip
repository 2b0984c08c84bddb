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
//   A = up to twelve tokens' activations of that block, fp16 high and low halves
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
//
// Batches of at most five and a half pairs per expert on average, with rows of up to 2048
// activations, take the integer matrix cores instead (moe_grouped_i8_kernel below: the digit
// planes of the few-token kernels, four tokens of an expert per product, operands in registers;
// its grouping step also cuts the pair lists into work items and lays out where each workgroup
// starts): they cost less per product and more per token, and win while most experts hold no
// more than a handful of pairs.
#include "moe_grouped.hpp"

#include <array>
#include <cstdio>
#include "q4_0_mfma.hpp"

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
// Activation planes.  A row is scaled by the power of two that brings its maximum into
// [2^14, 2^15) (zero, denormal and non-finite maxima: no scaling) and split into fp16 high and low
// halves.  At the top of fp16's range the low half of every element down to 2^-17 of the row's
// maximum is still a normal number: x = hi + lo to 2^-22 of the element (with the maximum in
// [1, 2) an element 2^-6 below it kept 18 bits, 2^-10 below it 14);
// run 4b + g of a row holds elements 4g, 4g+2, 4g+1, 4g+3, then 16+4g, 16+4g+2, 16+4g+1, 16+4g+3 of
// block b: the weights in code bytes 4g..4g+3 of the block (low nibbles, then high nibbles), in the
// order in which the masks of the matrix-core kernel deliver them.
// ---------------------------------------------------------------------------
struct grp_scale { float scale, unscale; };
__device__ __forceinline__ grp_scale grp_row_scale(uint32_t max_bits) {
    uint32_t ex = (max_bits >> 23) & 0xFFu;                    // maximum in [2^(ex - 127), 2^(ex - 126))
    if (ex == 0u || ex >= 254u) ex = 141u;                     // (no scaling)
    ex = ex < 15u ? 15u : ex;                                  // keeps both powers of two normal numbers
    return grp_scale{__uint_as_float((268u - ex) << 23), __uint_as_float((ex - 14u) << 23)};   // 2^(141 - ex), 2^(ex - 141)
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
                 uint32_t *__restrict__ xmax, uint32_t *__restrict__ amax, lev_grp_item *items,
                 uint32_t item_pairs, lev_grp_start *__restrict__ starts, uint32_t grid, uint32_t rpi_gu,
                 uint32_t rpi_dn, uint32_t w1_gu, uint32_t w2_gu, uint32_t w1_dn, uint32_t w2_dn, uint32_t s0_gu,
                 uint32_t s0_dn) {
    // [experts] counts | cursors | with items: first pair | first item of more than four pairs | first other item
    extern __shared__ int32_t s_cnt[];
    int32_t *s_cur = s_cnt + experts, *s_first = s_cur + experts, *s_big = s_first + experts, *s_small = s_big + experts;
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
    if (amax)
        for (uint32_t p = tid; p < pairs; p += 1024u) amax[p] = 0u;
    for (uint32_t e = tid; e < experts; e += 1024u) s_cnt[e] = 0;
    __syncthreads();
    bool bad_seen = false;
    int32_t e_own = -1;                          // the thread's first pair, kept for the placement: its expert, or -1
    for (uint32_t p = tid; p < pairs; p += 1024u) {
        const int32_t e = ids[p];
        bool ok = e >= 0 && (uint32_t)e < experts;
        const uint32_t slot = p % top_k, first = p - slot;
        // both copies of a duplicate are dropped; the token's ids are requested eight at a time (one
        // wait for eight, not one after the other)
        for (uint32_t k0 = 0; k0 < top_k; k0 += 8u) {
            int32_t other[8];
#pragma unroll
            for (uint32_t u = 0; u < 8u; ++u) other[u] = ids[first + (k0 + u < top_k ? k0 + u : slot)];
#pragma unroll
            for (uint32_t u = 0; u < 8u; ++u)
                if (k0 + u < top_k && k0 + u != slot && other[u] == e) ok = false;
        }
        valid[p] = ok ? 1 : 0;
        if (ok) atomicAdd(&s_cnt[e], 1);
        if (p == tid && ok) e_own = e;
        bad_seen = bad_seen || !ok;
    }
    if (bad_seen) atomicOr(flag, kFlagBadExpertId);
    __syncthreads();
    // exclusive scan of the counts (experts <= 4096): thread i takes experts 4i..4i+3, the waves scan
    // their threads' sums by shuffles and meet in LDS.  One scan carries three counts of at most
    // 2^20 each in 21-bit fields: pairs, items of more than four pairs, other items.
    __shared__ uint64_t s_wave[16];
    uint32_t n_big = 0u, n_all = 0u;            // items of more than four pairs, all items
    {
        int32_t c4[4], big4[4], small4[4];
        const int32_t ip = items ? (int32_t)item_pairs : 1, ish = ip == 8 ? 3 : ip == 4 ? 2 : 0;   // (4 or 8 pairs an item)
        uint64_t local = 0;
#pragma unroll
        for (uint32_t k = 0; k < 4u; ++k) {
            const uint32_t e = 4u * tid + k;
            c4[k] = e < experts ? s_cnt[e] : 0;
            // work items of the integer matrix-core kernels: runs of at most item_pairs pairs of one expert
            const int32_t full = c4[k] >> ish, rem = c4[k] - (full << ish);
            big4[k] = items ? (ip > 4 ? full : 0) + (rem > 4 ? 1 : 0) : 0;
            small4[k] = items ? (ip > 4 ? 0 : full) + (rem > 0 && rem <= 4 ? 1 : 0) : 0;
            local += (uint64_t)c4[k] | (uint64_t)big4[k] << 21 | (uint64_t)small4[k] << 42;
        }
        uint64_t incl = local;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const uint64_t o = __shfl_up(incl, off);
            if ((int)(tid & 63u) >= off) incl += o;
        }
        if ((tid & 63u) == 63u) s_wave[tid >> 6] = incl;
        __syncthreads();
        uint64_t before = incl - local, all = 0;
#pragma unroll
        for (uint32_t w = 0; w < 16u; ++w) {
            const uint64_t v = s_wave[w];
            before += w < (tid >> 6) ? v : 0u;
            all += v;
        }
        int32_t run = (int32_t)(before & 0x1FFFFFu);
        const int32_t first_pair = run;
#pragma unroll
        for (uint32_t k = 0; k < 4u; ++k) {
            const uint32_t e = 4u * tid + k;
            if (e <= experts) goff[e] = run;
            if (e < experts) s_cur[e] = run;
            run += c4[k];
        }
        // 4096 experts: the total has no thread of its own (thread i owns 4i..4i+3 <= 4095)
        if (4u * tid + 4u == experts && experts == 4096u) goff[experts] = run;
        if (items) {
            // Items of more than four pairs (two products a block) come first, in expert order, the
            // others behind them: what a round costs then depends on its position in the line of
            // rounds alone.
            const int32_t nbig = (int32_t)(all >> 21 & 0x1FFFFFu), nsmall = (int32_t)(all >> 42);
            int32_t brun = (int32_t)(before >> 21 & 0x1FFFFFu), srun = nbig + (int32_t)(before >> 42);
            n_big = (uint32_t)nbig;
            n_all = (uint32_t)(nbig + nsmall);
            int32_t prun = first_pair;
#pragma unroll
            for (uint32_t k = 0; k < 4u; ++k) {
                const uint32_t e = 4u * tid + k;
                if (e < experts) {
                    s_first[e] = prun;
                    s_big[e] = brun;
                    s_small[e] = srun;
                }
                const int32_t n = big4[k] + small4[k];
                for (int32_t j = 0; j < n; ++j) {
                    const int32_t left = c4[k] - j * ip, count = left < ip ? left : ip;
                    lev_grp_item *it = items + (count > 4 ? brun++ : srun++);
                    it->expert = (int32_t)e;
                    it->count = count;
                    it->first = prun + j * ip;
                }
                prun += c4[k];
            }
        }
    }
    __syncthreads();
    const uint32_t sid = 1023u - tid;   // (the high threads: the low ones place the first 1024 pairs below)
    if (items && sid < 2u * grid) {
        // Where the workgroups of the two expert kernels start.  A round of an item of more than
        // four pairs costs w2, any other w1, and beginning an item (its header, its activations,
        // their staging) costs s0 wherever the item begins; the line of items is cut into
        // stretches of equal COST.  The items of more than four pairs come first, so a position in
        // cost is a position in rounds by a few divisions (32-bit arithmetic: cost < 2^29,
        // grid <= 2^9).
        const uint32_t down = sid >= grid ? 1u : 0u, L = sid - down * grid, rpi = down ? rpi_dn : rpi_gu;
        const uint32_t w1 = down ? w1_dn : w1_gu, w2 = down ? w2_dn : w2_gu, s0 = down ? s0_dn : s0_gu;
        const uint32_t I2 = s0 + rpi * w2, I1 = s0 + rpi * w1;       // cost of a whole item
        const uint32_t R2 = n_big * rpi, C2 = n_big * I2;
        const uint32_t total = C2 + (n_all - n_big) * I1, per = total / grid, rest = total - per * grid;
        // rounds that lie wholly or partly before cost position c
        auto rounds_before = [&](uint32_t c) {
            const bool big = c <= C2;
            const uint32_t cc = big ? c : c - C2, I = big ? I2 : I1, w = big ? w2 : w1;
            const uint32_t item = cc / I, in_item = cc - item * I;
            const uint32_t r = in_item <= s0 ? 0u : (in_item - s0 + w - 1u) / w;
            return (big ? 0u : R2) + item * rpi + r;
        };
        lev_grp_start st;
        st.first_round = rounds_before(per * L + rest * L / grid);
        st.end_round = rounds_before(per * (L + 1u) + rest * (L + 1u) / grid);
        st.item = st.first_round / rpi;
        const lev_grp_item *it = items + (st.item < n_all ? st.item : 0u);   // (written before the barrier)
        st.expert = it->expert;
        st.count = it->count;
        st.pad[0] = st.pad[1] = st.pad[2] = 0u;
        starts[sid] = st;
    }
    // The order of an expert's pairs in the list depends on the atomics; no
    // result does: every pair is computed independently and owns its outputs.
    for (uint32_t p = tid; p < pairs; p += 1024u)
        if (p == tid ? e_own >= 0 : valid[p] != 0) {
            const int32_t e = p == tid ? e_own : ids[p];
            const int32_t at = atomicAdd(&s_cur[e], 1);
            glist[at] = (int32_t)p;
            if (items) {
                // the pair's column in its item: the expert's items of more than four pairs come
                // first in the expert's list (whole items, then a remainder of more than four)
                const int32_t ip = (int32_t)item_pairs, ish = ip == 8 ? 3 : 2, c = s_cnt[e], pos = at - s_first[e];
                const int32_t full = c >> ish, rem = c - (full << ish), nbig = (ip > 4 ? full : 0) + (rem > 4 ? 1 : 0);
                const int32_t j = pos >> ish;
                lev_grp_item *it = items + (j < nbig ? s_big[e] + j : s_small[e] + (j - nbig));
                const int32_t left = c - j * ip, count = left < ip ? left : ip, col = pos - j * ip;
                it->pair[col] = (int32_t)p;
                it->src[col] = (int32_t)(p / top_k);
                if (col == count - 1)   // the columns past the count repeat the last pair
                    for (int32_t k = count; k < 8; ++k) {
                        it->pair[k] = (int32_t)p;
                        it->src[k] = (int32_t)(p / top_k);
                    }
            }
        }
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
                m = lev_row16_max_u32(m);
                const uint32_t col = 4u * g + (uint32_t)i;
                if (r == 0u && col < ncols && m != 0u) atomicMax(out_max + s_pair[col], m);
            }
        }
    }
}

// ---------------------------------------------------------------------------
// 2./3. on the integer matrix cores, four tokens of an expert per product.
//
// v_mfma_i32_16x16x32_i8 multiplies 16 A rows x 32 k x 16 weight rows: ONE Q4_0 block of 16 weight
// rows.  A row 4t + p is digit plane p of token t (x as integers X = rint(x * 2^(156 - ex)), ex
// the exponent of the largest magnitude among the task's 256 activations, cut into four balanced
// base-256 digits: the arithmetic of the few-token kernels), so the output lane (row, t) holds
// the four plane sums of token t against its row's block: they are recombined in 32-bit integers
// and f32 and scaled by the block's d there, with nothing exchanged between lanes.  B: lane
// (row, g) supplies code bytes 4g..4g+3 of the block, low nibbles then high nibbles, as int8
// 16 * (n - 8) (flip the top bit of every nibble, mask; the low nibbles shifted up first).
//
// A task is fetched as in the decode GEMV (a quad of lanes reads the 144 contiguous bytes of a
// row's four block pairs; one lane permutation per dword brings pair g of row r to lane (r, g));
// the dwords of a block are then spread over the four lanes of its row by a 4 x 4 transpose
// between the lane groups (four row swaps), and the scales of the row's eight blocks are
// gathered the same way.
//
// A work ITEM is up to kG8NT pairs of one expert (the grouping kernel cuts each expert's list into
// such runs).  Every item takes the same number of ROUNDS over its expert's rows, so the rounds of
// all items form one line that the grid's workgroups cut into equal stretches, whatever the
// routing: a workgroup works through `total * L / G .. total * (L + 1) / G` and stages the
// activations of each item its stretch touches.  Stretches that follow each other go to
// workgroups of one XCD (an expert with more than kG8NT pairs is streamed by neighbours, through
// one L2).
//
// Workgroup = wpr * slots waves (eight for gate/up, twelve for down), as in the decode GEMV: wave (slot, pos) owns
// column task `pos` (256 activations) of the row groups of its slot, stages the task's
// activations for all of the item's tokens by itself and keeps the operands in registers (16 per
// four tokens).  A round of a wave is NTILE tiles of 16 rows x 256 codes: gate and up rows of one
// row group (PAIRED), or NTILE consecutive row groups (down); the next round's bytes are
// requested as soon as this round's have been handed to the lanes that multiply them.  The wpr
// partial sums of a (row, token) meet in LDS behind one barrier a batch of rounds; wave u adds
// unit u of the batch (a slot's 16 rows x four tokens), applies the activation function (PAIRED)
// and stores.
// ---------------------------------------------------------------------------
constexpr uint32_t kG8MaxGrid = 512;                      // workgroups of an expert kernel (one per CU)
constexpr int kG8MaxWpr = 8;                              // waves that share a row group: one task each
constexpr int kG8WavesGateUp = 8;                         // 2048 activations: eight column tasks, one slot
constexpr int kG8WavesDown = 12;                          // 768 activations: three column tasks, four slots (three
                                                          // waves a SIMD; eight waves leave two SIMDs with one)
constexpr int kG8TilesDown = 1;                          // row groups a wave of the down kernel takes per round (2: rounds twice
                                                          // as long, the stretches a workgroup gets then differ by more: 106.8
                                                          // against 104.4 us a layer at 64 tokens)
constexpr int kG8NT = 8;                                  // tokens per item
static_assert(kG8NT == 4 || kG8NT == 8, "an item is one or two groups of four tokens");
constexpr uint32_t kG8Batch = 4;                          // rounds between two barriers of a workgroup (2: 55.4
                                                          // against 53.6 us for gate/up, 1: 64.9)
constexpr uint32_t kG8MaxInLen = 256u * kG8MaxWpr;
constexpr uint32_t kG8Plane = 272u;                       // a digit plane of a staged task: 256 bytes + 16, so that
constexpr uint32_t kG8TokArea = 4u * kG8Plane;            // the 64 lanes of an operand read hit 64 different banks
constexpr uint32_t kG8WaveLds = 4u * kG8TokArea;           // four tokens are staged at a time

// LDS: part [parity 2][round of the batch][tile NTILE][token group of the item][wave][row 16][token % 4] f32 | per
// wave four staged tasks
template <int NTILE, int NW>
constexpr size_t g8_lds() {
    return (size_t)2 * kG8Batch * NTILE * (kG8NT / 4) * (NW * 256u) + (size_t)NW * kG8WaveLds;
}

// Digit planes of one token's task into `tok` (kG8TokArea bytes, this wave's own): lane i holds
// elements 4i..4i+3 of the task's 256 activations; plane p, byte e = digit p of element e.
// Returns the power of two that undoes the scaling (and the 16 of the codes); NaN when the task
// holds a NaN or an infinity.
__device__ __forceinline__ float g8_stage_token(const lev_f32x4 v, uint8_t *tok) {
    const uint32_t lane = threadIdx.x & 63u;
    uint32_t mb = 0u;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const uint32_t bits = __float_as_uint(v[k]) & 0x7FFFFFFFu;
        mb = bits > mb ? bits : mb;
    }
    mb = lev_wave_max_u32(mb);   // every lane: the task's maximum
    uint32_t ex = mb >> 23;                                    // |x| < 2^(ex - 126)
    const bool bad = ex == 255u;
    ex = ex < 34u ? 34u : (ex > 254u ? 254u : ex);             // keeps both powers of two normal numbers
    const float scale = __uint_as_float((283u - ex) << 23);    // 2^(156 - ex): |x * scale| < 2^30
    uint32_t Y[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) Y[k] = ((uint32_t)(int)rintf(v[k] * scale) + 0x00808080u) ^ 0x00808080u;
    // 4x4 byte transpose: digit p of the lane's four values in one dword
    const uint32_t t0 = __builtin_amdgcn_perm(Y[1], Y[0], 0x05010400u);
    const uint32_t t1 = __builtin_amdgcn_perm(Y[1], Y[0], 0x07030602u);
    const uint32_t t2 = __builtin_amdgcn_perm(Y[3], Y[2], 0x05010400u);
    const uint32_t t3 = __builtin_amdgcn_perm(Y[3], Y[2], 0x07030602u);
    uint32_t *at = reinterpret_cast<uint32_t *>(tok + 4u * lane);
    at[0u * (kG8Plane / 4u)] = __builtin_amdgcn_perm(t2, t0, 0x05040100u);
    at[1u * (kG8Plane / 4u)] = __builtin_amdgcn_perm(t2, t0, 0x07060302u);
    at[2u * (kG8Plane / 4u)] = __builtin_amdgcn_perm(t3, t1, 0x05040100u);
    at[3u * (kG8Plane / 4u)] = __builtin_amdgcn_perm(t3, t1, 0x07060302u);
    return bad ? __builtin_nanf("") : __uint_as_float((ex - 33u) << 23);   // 2^(ex - 160)
}

// A operands of four staged tokens (`toks`: their kG8TokArea areas, one behind the other): lane
// (a, g) = (lane % 16, lane / 16) supplies, for block b of the task, plane a % 4 of token a / 4
// at the block's elements 4g..4g+3 and 16+4g..16+4g+3 (the elements whose codes lie in bytes
// 4g..4g+3 of the block).
__device__ __forceinline__ void g8_read_operands(const uint8_t *toks, long (&A)[8]) {
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t a = lane & 15u, g = lane >> 4;
    const uint32_t *p = reinterpret_cast<const uint32_t *>(toks + (a >> 2) * kG8TokArea + (a & 3u) * kG8Plane + 4u * g);
#pragma unroll
    for (int b = 0; b < 8; ++b) A[b] = (long)(((uint64_t)p[8 * b + 4] << 32) | (uint64_t)p[8 * b]);
}

// In: lane (r, g) holds q[j] = dword j of a record of lane group g.  Out: q[P] = dword g of the
// record of lane group P (a 4 x 4 transpose between the four lanes of a row, by row swaps).
__device__ __forceinline__ void g8_transpose4(uint32_t (&q)[4]) {
    const auto a = __builtin_amdgcn_permlane16_swap(q[0], q[1], false, false);
    const auto b = __builtin_amdgcn_permlane16_swap(q[2], q[3], false, false);
    const auto c = __builtin_amdgcn_permlane32_swap(a[0], b[0], false, false);
    const auto d = __builtin_amdgcn_permlane32_swap(a[1], b[1], false, false);
    q[0] = c[0]; q[1] = d[0]; q[2] = c[1]; q[3] = d[1];
}

// One tile (16 rows x 256 codes; W: the lane's pair, already turned) against NJ groups of four
// tokens, of which the first ng take part: val[j] = the task's sum for (row lane % 16, token
// 4j + lane / 16), blocks added in their order.
template <uint32_t NJ>
__device__ __forceinline__ void g8_tile_dot(const uint32_t W[9], const long (&A)[NJ][8], uint32_t ng,
                                            const float (&unscale)[NJ], float (&val)[NJ]) {
    uint32_t qa[4], qb[4];
    qa[0] = __builtin_amdgcn_alignbit(W[1], W[0], 16);
    qa[1] = __builtin_amdgcn_alignbit(W[2], W[1], 16);
    qa[2] = __builtin_amdgcn_alignbit(W[3], W[2], 16);
    qa[3] = __builtin_amdgcn_alignbit(W[4], W[3], 16);
    qb[0] = W[5]; qb[1] = W[6]; qb[2] = W[7]; qb[3] = W[8];
    g8_transpose4(qa);
    g8_transpose4(qb);
    // the pair's two scales in one dword, then every lane of a row gets the row's four dwords
    const uint32_t dd = __builtin_amdgcn_perm(W[4], W[0], 0x07060100u);
    const auto s = __builtin_amdgcn_permlane16_swap(dd, dd, false, false);      // pairs g & ~1, g | 1
    const auto e = __builtin_amdgcn_permlane32_swap(s[0], s[0], false, false);  // pairs 0, 2
    const auto o = __builtin_amdgcn_permlane32_swap(s[1], s[1], false, false);  // pairs 1, 3
    const uint32_t dp[4] = {e[0], o[0], e[1], o[1]};
    long B[8];
    float d[8];
#pragma unroll
    for (int b = 0; b < 8; ++b) {
        const uint32_t q = ((b & 1) ? qb[b >> 1] : qa[b >> 1]) ^ 0x88888888u;
        B[b] = (long)(((uint64_t)(q & 0xF0F0F0F0u) << 32) | (uint64_t)((q << 4) & 0xF0F0F0F0u));
        d[b] = lev_f16_bits_to_f32((b & 1) ? dp[b >> 1] >> 16 : dp[b >> 1] & 0xFFFFu);
    }
    // a group's eight products are independent: they issue back to back, the sums follow
    auto group = [&](const long (&Aj)[8]) {
        lev_i32x4 acc[8];
#pragma unroll
        for (int b = 0; b < 8; ++b)
            acc[b] = __builtin_amdgcn_mfma_i32_16x16x32_i8(Aj[b], B[b], lev_i32x4{0, 0, 0, 0}, 0, 0, 0);
        float v = 0.f;
#pragma unroll
        for (int b = 0; b < 8; ++b) {
            // |plane sum| <= 32 * 128 * 128 = 2^19: two planes recombine in 32 bits, the halves in f32
            const float f = fmaf((float)(acc[b][2] + (acc[b][3] << 8)), 65536.0f, (float)(acc[b][0] + (acc[b][1] << 8)));
            v = fmaf(d[b], f, v);
        }
        return v;
    };
    val[0] = group(A[0]);
#pragma unroll
    for (uint32_t j = 1; j < NJ; ++j) {
        val[j] = 0.f;
        if (j < ng) val[j] = group(A[j]);
    }
#pragma unroll
    for (uint32_t j = 0; j < NJ; ++j) val[j] *= unscale[j];
}

template <int NTILE, bool PAIRED, int NW>
__global__ void __launch_bounds__(NW * LEV_WAVE)
moe_grouped_i8_kernel(lev_moe_grouped_args a, const float *__restrict__ src, const lev_grp_item *__restrict__ items,
                      const lev_grp_start *__restrict__ starts, float *__restrict__ out, uint32_t wpr, uint32_t slots,
                      uint32_t rpi, uint64_t slot_of_wave, uint64_t pos_of_wave) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    constexpr uint32_t NT = kG8NT, NJ = NT / 4u;
    constexpr uint32_t TO = PAIRED ? 1u : (uint32_t)NTILE;       // row groups a slot finishes per round
    constexpr uint32_t kG8Unit = NW * 256u;                       // bytes of part[wave][row][token % 4]: one tile's sums of four tokens
    constexpr uint32_t kHalf = kG8Batch * NTILE * NJ * kG8Unit;   // one parity of `part`: a batch of rounds (with one
                                                                  // token group an item: twice as many rounds)
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const uint32_t nwaves = blockDim.x >> 6;                      // wpr * slots: every wave has a task
    const uint32_t slot = (uint32_t)(slot_of_wave >> (4u * wave)) & 15u;
    const uint32_t tw = (uint32_t)(pos_of_wave >> (4u * wave)) & 15u;
    const uint32_t in_len = PAIRED ? a.hidden : a.inter, out_rows = PAIRED ? a.inter : a.hidden;
    const uint32_t ngroups = (out_rows + 15u) >> 4;
    const uint64_t row_bytes = (uint64_t)(in_len >> 6) * 36u;
    const uint32_t r = lane & 15u, g = lane >> 4, lrow = lane >> 2;

    // this workgroup's stretch of the line of rounds
    const uint32_t G = gridDim.x;
    const uint32_t L = (G & 7u) == 0u ? (blockIdx.x & 7u) * (G >> 3) + (blockIdx.x >> 3) : blockIdx.x;
    // (stretches of equal cost, laid out by the grouping kernel together with the first item's header)
    const lev_grp_start st = starts[L];
    uint32_t R = st.first_round, it = st.item;
    const uint32_t Rend = st.end_round;
    uint32_t e = (uint32_t)st.expert, cnt = (uint32_t)st.count;

    uint8_t *area = smem + 2u * kHalf + (size_t)wave * kG8WaveLds;
    // byte offsets into the workgroup's LDS, not pointers; lane (r, g) writes row r, token 4j + g
    uint32_t pw = ((wave * 16u + r) * 4u + g) * 4u;
    uint32_t half = 0u;                                           // byte offset of the round's parity

    while (R < Rend) {
        const uint32_t r0 = R - it * rpi;
        const uint32_t nr = rpi - r0 < Rend - R ? rpi - r0 : Rend - R;   // rounds r0 .. r0 + nr of item `it`
        // request order = return order: the item's columns (scalar loads), the activations of the
        // wave's task for every token, and the first round's weights behind them, so that the
        // staging does not wait for the weights.  The header of the NEXT item is requested here as
        // well (the list has one record past its end): its expert is known when its turn comes.
        const lev_grp_item *item = items + it;
        const uint32_t e_next = (uint32_t)item[1].expert, cnt_next = (uint32_t)item[1].count;
        const uint32_t ng = (cnt + 3u) >> 2;                      // groups of four tokens that take part
        int32_t pk[NT];
        lev_f32x4 v[NT];
#pragma unroll
        for (uint32_t k = 0; k < NT; ++k) {
            pk[k] = item->pair[k];
            const uint32_t srow = (uint32_t)(PAIRED ? item->src[k] : item->pair[k]);
            v[k] = reinterpret_cast<const lev_f32x4 *>(src + (uint64_t)srow * in_len)[64u * tw + lane];
        }
        const uint8_t *m0 = a.base + (PAIRED ? a.gate_off + e * a.gate_stride : a.down_off + e * a.down_stride);
        const uint8_t *m1 = PAIRED ? a.base + a.up_off + e * a.up_stride : m0;
        auto issue = [&](uint32_t rho, uint32_t (&D)[NTILE][9]) {
#pragma unroll
            for (int t = 0; t < NTILE; ++t) {
                uint32_t rg = PAIRED ? rho * slots + slot : (rho * slots + slot) * (uint32_t)NTILE + (uint32_t)t;
                rg = rg < ngroups ? rg : ngroups - 1u;
                uint32_t row = rg * 16u + lrow;
                row = row < out_rows ? row : out_rows - 1u;
                q4m_load_task((PAIRED && t == 1 ? m1 : m0) + (uint64_t)row * row_bytes, 4u * tw, D[t]);
            }
        };
        __builtin_amdgcn_sched_barrier(0);
        const uint32_t r_last = r0 + nr - 1u;
        uint32_t Da[NTILE][9];
        issue(r0, Da);
        __builtin_amdgcn_sched_barrier(0);
        // the activations are requested for every column, whatever the item's count (columns past
        // the count repeat the last pair), in front of the weights: a request inside the branch
        // below would queue behind them
#pragma unroll
        for (uint32_t k = 0; k < NT; ++k) lev_pin(v[k]);
        long A[NJ][8];
        float unscale[NJ];
#pragma unroll
        for (uint32_t j = 0; j < NJ; ++j) {
#pragma unroll
            for (int b = 0; b < 8; ++b) A[j][b] = 0;
            unscale[j] = 0.f;
            if (j < ng) {
                // the area belongs to this wave alone: LDS runs a wave's accesses in order, the fences
                // only keep the compiler from moving reads above writes (and the next group's writes
                // above these reads)
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                float us[4];
#pragma unroll
                for (uint32_t k = 0; k < 4u; ++k) us[k] = g8_stage_token(v[4u * j + k], area + k * kG8TokArea);
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                g8_read_operands(area, A[j]);
                unscale[j] = g == 0u ? us[0] : g == 1u ? us[1] : g == 2u ? us[2] : us[3];
            }
        }
        // the operands are read back before the wait for the weights, not behind it
        __builtin_amdgcn_sched_barrier(0);

        uint32_t batch0 = r0, nb = 0u;                            // the batch's first round, rounds in it so far
        const uint32_t round_bytes = NTILE * ng * kG8Unit;        // one round's sums in `part`: [tile][token group][wave][row][token % 4]
        const uint32_t batch_rounds = kG8Batch * NJ / ng;
        auto round = [&](uint32_t rho, uint32_t (&D)[NTILE][9]) {
            // lane (r, g) <- lane 4r + g; the registers the bytes came in take a later round's
            // request at once (unconditional, clamped: a branch around the loads would make the
            // compiler wait for them before this round is multiplied)
            uint32_t W[NTILE][9];
#pragma unroll
            for (int t = 0; t < NTILE; ++t) q4m_turn_task(D[t], W[t]);
            __builtin_amdgcn_sched_barrier(0);
            issue(rho + 1u < r_last ? rho + 1u : r_last, D);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int t = 0; t < NTILE; ++t) {
                float val[NJ];
                g8_tile_dot<NJ>(W[t], A, ng, unscale, val);
#pragma unroll
                for (uint32_t j = 0; j < NJ; ++j)
                    if (j < ng)
                        *reinterpret_cast<float *>(smem + half + nb * round_bytes + pw + ((uint32_t)t * ng + j) * kG8Unit) = val[j];
            }
            // the waves meet once per batch of rounds (and at the item's end): between two barriers
            // they run at their own pace, and the batch's sums are finished by several waves at once
            if (++nb < batch_rounds && rho != r_last) return;
            lev_barrier_lds();
            // unit u = (round b of the batch, slot s, row group t of the slot's round, tokens 4j .. 4j + 3):
            // lane (r, g) adds the slot's waves' sums of row r and token 4j + g in a fixed order
            static_assert(NJ <= 2u, "the unit index is split by a shift");
            const uint32_t per_round = slots * TO * ng;
            for (uint32_t u = wave; u < nb * per_round; u += nwaves) {
                const uint32_t b = u / per_round, ur = u - b * per_round;
                const uint32_t j = ur & (ng - 1u), us_ = ur >> (ng - 1u), s = us_ / TO, t = us_ % TO;
                const uint32_t k = 4u * j + g;
                const uint32_t rg = PAIRED ? (batch0 + b) * slots + s : ((batch0 + b) * slots + s) * (uint32_t)NTILE + t;
                const uint32_t row = rg * 16u + r;
                const float *pp = reinterpret_cast<const float *>(
                    smem + half + b * round_bytes + (t * ng + j) * kG8Unit + ((s * wpr * 16u + r) * 4u + g) * 4u);
                auto slot_sum = [&](const float *q) {
                    float p[kG8MaxWpr];
#pragma unroll
                    for (uint32_t w = 0; w < (uint32_t)kG8MaxWpr; ++w) p[w] = q[(w < wpr ? w : 0u) * 64u];   // eight reads in flight
#pragma unroll
                    for (uint32_t w = 0; w < (uint32_t)kG8MaxWpr; ++w) p[w] = w < wpr ? p[w] : 0.f;
                    return ((p[0] + p[4]) + (p[2] + p[6])) + ((p[1] + p[5]) + (p[3] + p[7]));
                };
                float res = slot_sum(pp);
                if (PAIRED) res = lev_gelu_up_value(res, slot_sum(pp + ng * (kG8Unit / 4u)));
                int32_t pair = pk[0];
#pragma unroll
                for (uint32_t q = 1; q < NT; ++q) pair = k == q ? pk[q] : pair;
                if (k < cnt && row < out_rows) out[(uint64_t)(uint32_t)pair * out_rows + row] = res;
            }
            half ^= kHalf;
            batch0 = rho + 1u;
            nb = 0u;
        };
        for (uint32_t rho = r0; rho <= r_last; ++rho) round(rho, Da);
        R += nr;
        ++it;
        e = e_next;
        cnt = cnt_next;
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
    size_t goff, glist, valid, xh, xl, xmax, amax, dn, items, starts, total;
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
    L.items = o; o += align256((pairs / 8 + a.experts + 1) * sizeof(lev_grp_item));   // an expert with c pairs: ceil(c / 8) items; one past the end
    L.starts = o; o += 2 * kG8MaxGrid * sizeof(lev_grp_start);
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

// Where the integer matrix-core kernels serve: rows of whole 256-value tasks, one task per wave, and
// at most five and a half pairs per expert on average -- they multiply four tokens at a time and are
// the faster ones while most experts hold no more than four or eight pairs; the fp16 kernel above takes
// twelve tokens a pass at one price.  LEV_MOE_GROUPED_I8=0 keeps the fp16 kernel, =1 takes the
// integer kernels for any token count (for comparison and for the tests).
bool g8_usable(const lev_ctx *ctx, const lev_moe_grouped_args &a) {
    static const int mode = [] {
        const char *v = getenv("LEV_MOE_GROUPED_I8");
        return v && v[0] == '0' ? 0 : v && v[0] == '1' ? 1 : 2;
    }();
    if (mode == 0) return false;
    const bool shape = a.hidden % 256u == 0u && a.hidden <= kG8MaxInLen && a.inter % 256u == 0u && a.inter <= kG8MaxInLen;
    const size_t limit = ctx->props.sharedMemPerBlockOptin > ctx->props.sharedMemPerBlock
                             ? ctx->props.sharedMemPerBlockOptin
                             : ctx->props.sharedMemPerBlock;
    const size_t lds_group = (size_t)5 * a.experts * 4;
    const bool fits = g8_lds<2, kG8WavesGateUp>() <= limit && g8_lds<kG8TilesDown, kG8WavesDown>() <= limit && lds_group <= limit;
    // (64 tokens x top-8 over 128 experts, experts only, us: 72 tokens 106 against 119, 88 tokens 117 against 119,
    // 96 tokens 132 against 124)
    return shape && fits && (mode == 1 || 2u * (uint64_t)a.tokens * a.top_k <= 11u * (uint64_t)a.experts);
}

struct g8_geometry {
    uint32_t wpr, slots, rpi;   // waves a row, row-group slots a workgroup, rounds an item
};
template <int NTILE, bool PAIRED, int NW>
g8_geometry g8_geometry_of(const lev_moe_grouped_args &a) {
    const uint32_t in_len = PAIRED ? a.hidden : a.inter, out_rows = PAIRED ? a.inter : a.hidden;
    g8_geometry q;
    q.wpr = in_len >> 8;
    q.slots = (uint32_t)NW / q.wpr;
    const uint32_t ngroups = (out_rows + 15u) / 16u;
    const uint32_t per_round = q.slots * (PAIRED ? 1u : (uint32_t)NTILE);   // row groups a round finishes
    q.rpi = (ngroups + per_round - 1u) / per_round;
    return q;
}

template <int NTILE, bool PAIRED, int NW>
hipError_t g8_launch(lev_ctx *ctx, const lev_moe_grouped_args &a, const float *src, const lev_grp_item *items,
                     const lev_grp_start *starts, uint32_t grid, float *out) {
    const g8_geometry q = g8_geometry_of<NTILE, PAIRED, NW>(a);
    uint64_t slot_of_wave, pos_of_wave;
    lev_wave_tables(q.wpr, &slot_of_wave, &pos_of_wave);
    constexpr size_t lds = g8_lds<NTILE, NW>();
    static bool configured = false;   // per instantiation: raise the dynamic LDS limit once
    if (!configured) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&moe_grouped_i8_kernel<NTILE, PAIRED, NW>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        configured = true;
    }
    hipLaunchKernelGGL((moe_grouped_i8_kernel<NTILE, PAIRED, NW>), dim3(grid), dim3(64u * q.wpr * q.slots), lds,
                       ctx->stream, a, src, items, starts, out, q.wpr, q.slots, q.rpi, slot_of_wave, pos_of_wave);
    return hipGetLastError();
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

    if (g8_usable(ctx, a)) {
        lev_grp_item *items = reinterpret_cast<lev_grp_item *>(s + L.items);
        lev_grp_start *starts = reinterpret_cast<lev_grp_start *>(s + L.starts);
        const uint32_t grid = (uint32_t)ctx->num_cus < kG8MaxGrid ? (uint32_t)ctx->num_cus : kG8MaxGrid;
        const g8_geometry q_gu = g8_geometry_of<2, true, kG8WavesGateUp>(a), q_dn = g8_geometry_of<kG8TilesDown, false, kG8WavesDown>(a);
        // what a round of an item of up to four pairs and of a larger one cost, relative to each other
        // (gate/up 52 against 62 us, down 33 against 38 with every item of the one or the other kind;
        // equal weights: 62 + 39 us at 64 tokens, these: 58 + 36.5)
        // cost of a round of an item of at most four pairs / of more, and of beginning an item, per kernel.
        // Measured at 64 tokens over 128 experts, us a layer in alternating runs on one box: no cost of
        // beginning 106.4, with it 104.5; down rounds 10:12 103.5, 10:14 101.6, 10:16 103.4 (the items of more
        // than four pairs come first in the line and go to the first XCDs, which finished 8 % after the others
        // at 5:6); gate/up rounds 10:13 and 10:14 no better than 5:6.  Thirteen settings around these, five
        // alternating runs each: medians 101.4 to 103.7, these 102.0
        // (LEV_MOE_CUT="w1,w2,s0,w1,w2,s0", gate/up then down, each 1..64 resp. 0..256: other weights, for measurement)
        static const std::array<uint32_t, 6> cut = [] {
            std::array<uint32_t, 6> c = {5u, 6u, 12u, 10u, 14u, 24u};
            unsigned v[6];
            const char *e = getenv("LEV_MOE_CUT");
            if (e && sscanf(e, "%u,%u,%u,%u,%u,%u", &v[0], &v[1], &v[2], &v[3], &v[4], &v[5]) == 6 && v[0] >= 1u &&
                v[0] <= 64u && v[1] >= 1u && v[1] <= 64u && v[2] <= 256u && v[3] >= 1u && v[3] <= 64u && v[4] >= 1u &&
                v[4] <= 64u && v[5] <= 256u)
                for (int i = 0; i < 6; ++i) c[i] = v[i];
            return c;
        }();
        const uint32_t w1 = cut[0], w2 = cut[1], s0_gu = cut[2], w1_dn = cut[3], w2_dn = cut[4], s0_dn = cut[5];
        const size_t lds_group = (size_t)5 * a.experts * 4;
        static size_t lds_group_set = 0;
        if (lds_group > 48 * 1024 && lds_group > lds_group_set) {
            e = hipFuncSetAttribute(reinterpret_cast<const void *>(&moe_group_kernel),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_group);
            if (e != hipSuccess) return e;
            lds_group_set = lds_group;
        }
        hipLaunchKernelGGL(moe_group_kernel, dim3(1), dim3(1024), lds_group, ctx->stream, ids, pairs,
                           a.experts, a.top_k, goff, glist, valid, ctx->d_flag, x, a.hidden, nullptr, nullptr, nullptr,
                           nullptr, items, (uint32_t)kG8NT, starts, grid, q_gu.rpi, q_dn.rpi, w1, w2, w1_dn, w2_dn,
                           s0_gu, s0_dn);
        if ((e = hipGetLastError()) != hipSuccess) return e;
        if ((e = g8_launch<2, true, kG8WavesGateUp>(ctx, a, x, items, starts, grid, act)) != hipSuccess) return e;
        // rows of act that belong to dropped pairs are never written and never read
        if ((e = g8_launch<kG8TilesDown, false, kG8WavesDown>(ctx, a, act, items, starts + grid, grid, dn)) != hipSuccess) return e;
        hipLaunchKernelGGL(moe_merge_kernel, dim3((a.hidden + 1023) / 1024, a.tokens), dim3(256), 0, ctx->stream, dn,
                           weights, valid, y, a.hidden, a.top_k);
        return hipGetLastError();
    }
    hipLaunchKernelGGL(moe_group_kernel, dim3(1 + a.tokens), dim3(1024), (size_t)2 * a.experts * 4,
                       ctx->stream, ids, pairs, a.experts, a.top_k, goff, glist, valid, ctx->d_flag, x,
                       a.hidden, xh, xl, xmax, amax, nullptr, 0u, nullptr, 0u, 0u, 0u, 0u, 0u, 0u, 0u, 0u, 0u);
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

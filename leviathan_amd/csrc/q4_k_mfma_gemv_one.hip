// (RMSNorm +) Q4_K GEMV for ONE column of f32 activations on the integer matrix cores (gfx950),
// for rows of at most sixteen superblocks.
//
// Stands in for Builder::norm_quant + Builder::matvec at one column
// (rust/crates/lev-model/src/gpu.rs:295, 334-370; q4k.matvec, lev-forge/src/glsl.rs:157-281),
// with the arithmetic of q4_k_mfma_gemv.hip (exact integer sums per sub-block, f64 behind them)
// in the shape of the Q4_0 decode kernel (q4_0_mfma_gemv.hip): a wave owns ONE superblock
// column of the matrix.  It stages the 256 activations of that column by itself, keeps the
// operands in registers and walks the row groups of its slot with the next groups' weights in
// flight, so that nothing but the RMSNorm's sum of squares crosses waves before the products.
//
// A superblock of a row (144 bytes: d, dmin, 12 bytes of 6-bit scales and mins, 128 bytes of
// codes; w = d*sc_j*q - dmin*m_j, rust/crates/lev-cpu/src/lib.rs:111-154) is four chunks of 32
// code bytes: low nibbles = sub-block 2c, high nibbles = sub-block 2c+1.  Lane (r, g) of the
// matrix core multiplies chunk g of row r: four v_mfma_i32_16x16x64_i8, two per sub-block, A row
// 4g + p holding digit plane p of the 16 activations lane group g multiplies and zeros elsewhere
// (see q4_0_mfma.hpp).  Low nibbles go in as q, high nibbles as 16*(q - 8) (mask and flip, one
// operation per four codes); the 8 comes back as 128 * (sum of the plane's digits), known per wave.
//
//   y += 2^e * ( d * sum_j sc_j * sum_k q_k X_k  -  dmin * sum_j m_j * sum_k X_k ),
//   X = rint(x * 2^-e) with |X| <= 2^25 per superblock, in four balanced base-256 digits.
// The sums over k are exact (32-bit integers); planes, d, dmin and 2^e are applied in f64, the
// partial sums of a row are added in f64 in a fixed order and rounded to f32 once.
//
// Weight bytes are fetched with the four chunks of a row's superblock in four ADJACENT lanes
// (lane 4*row + c: dword c of the header and the 32 aligned bytes of chunk c; a quad reads the
// row's 144 contiguous bytes) and handed to the lane the matrix core wants them in by one lane
// permutation per dword.  With lane (r, g) fetching for itself every lane of a quad is on another
// row, and with 36-byte quarters through a turn-round area in LDS the same kernel took 9.1 us
// instead of 7.9 at 12288 x 4096.
#include "q4_0_mfma.hpp"

namespace {

constexpr int kOneWaves = 16;
constexpr int kOneThreads = kOneWaves * LEV_WAVE;
// LDS for NC columns: part [2][16 waves][16 rows][NC] f64 | sums of squares [NC][16] f64 | per
// wave: NC staging areas of its activations, a zero strip
__host__ __device__ constexpr uint32_t q4k_one_part_bytes(uint32_t nc) { return 2u * kOneWaves * 16u * 8u * nc; }
__host__ __device__ constexpr uint32_t q4k_one_norm_bytes(uint32_t nc) { return kOneWaves * 8u * nc; }
__host__ __device__ constexpr uint32_t q4k_one_wave_bytes(uint32_t nc) { return nc * kQ4mTaskArea + kQ4mZeroBytes; }
__host__ __device__ constexpr size_t q4k_one_lds(uint32_t nc) {
    return q4k_one_part_bytes(nc) + q4k_one_norm_bytes(nc) + (size_t)kOneWaves * q4k_one_wave_bytes(nc);
}

// What a lane keeps of one column of its wave's 256 activations besides the digit planes.
struct q4k_one_column {
    int c1[4];          // 128 * (sum of plane p's digits over the high sub-block): undoes the -8 of its codes
    double sx0, sx1;    // sum of X over the low / high sub-block
    double ps;          // 2^(e - 4): undoes the scaling and the 16 of the codes; 0 for an idle wave, NaN for bad input
};

#define LEV_Q4K1_DPP(v, CTRL) __builtin_amdgcn_update_dpp(0, (v), (CTRL), 0xF, 0xF, true)

// Stages the wave's 256 activations of one column (lane i: elements 4i .. 4i+3) as digit planes
// [chunk 4][plane 4][half 4][16 B] in `area` (1 KB, the wave's own).
__device__ __forceinline__ void q4k_one_stage(const lev_f32x4 v, uint8_t *area, bool live, q4k_one_column &op) {
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t r = lane & 15u, g = lane >> 4;
    uint32_t mb = 0u;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const uint32_t bits = __float_as_uint(v[k]) & 0x7FFFFFFFu;
        mb = bits > mb ? bits : mb;
    }
    // one power of two per superblock, as in the kernels for several columns: the same integers,
    // so a column gives the same bits whichever kernel multiplies it
    mb = lev_wave_max_u32(mb);
    uint32_t ex = mb >> 23;                                    // |x| < 2^(ex - 126)
    const bool bad = ex == 255u;                               // NaN or infinity among the 256
    ex = ex < 25u ? 25u : (ex > 254u ? 254u : ex);             // keeps both powers of two normal numbers
    const float scale = __uint_as_float((278u - ex) << 23);    // 2^(151 - ex): |x * scale| < 2^25
    const double ps = __hiloint2double((int)((ex + 868u) << 20), 0);   // 2^(ex - 155)
    op.ps = !live ? 0.0 : bad ? (double)__builtin_nanf("") : ps;
    int X[4], sum = 0;
    uint32_t Y[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        X[k] = (int)rintf(v[k] * scale);
        sum += X[k];
        Y[k] = ((uint32_t)X[k] + 0x00808080u) ^ 0x00808080u;   // bytes = balanced base-256 digits
    }
    // 4x4 byte transpose: digit p of the lane's four values in one dword
    const uint32_t t0 = __builtin_amdgcn_perm(Y[1], Y[0], 0x05010400u);
    const uint32_t t1 = __builtin_amdgcn_perm(Y[1], Y[0], 0x07030602u);
    const uint32_t t2 = __builtin_amdgcn_perm(Y[3], Y[2], 0x05010400u);
    const uint32_t t3 = __builtin_amdgcn_perm(Y[3], Y[2], 0x07030602u);
    uint32_t dw[4];
    dw[0] = __builtin_amdgcn_perm(t2, t0, 0x05040100u);
    dw[1] = __builtin_amdgcn_perm(t2, t0, 0x07060302u);
    dw[2] = __builtin_amdgcn_perm(t3, t1, 0x05040100u);
    dw[3] = __builtin_amdgcn_perm(t3, t1, 0x07060302u);
    // sums over a sub-block = the eight lanes of half a row of 16
    int ps4[4];
#pragma unroll
    for (int p = 0; p < 4; ++p) ps4[p] = __builtin_amdgcn_sdot4((int)dw[p], 0x01010101, 0, false);
#define LEV_Q4K1_HALFROW(v)            \
    v += LEV_Q4K1_DPP(v, 0xB1);        \
    v += LEV_Q4K1_DPP(v, 0x4E);        \
    v += LEV_Q4K1_DPP(v, 0x141);
    LEV_Q4K1_HALFROW(sum)
#pragma unroll
    for (int p = 0; p < 4; ++p) { LEV_Q4K1_HALFROW(ps4[p]) }
#undef LEV_Q4K1_HALFROW
    const bool upper = (lane & 8u) != 0u;                      // this lane staged part of the high sub-block
    const int other = __builtin_amdgcn_update_dpp(0, sum, 0x140, 0xF, 0xF, true);   // row_mirror: the other half's sum
    op.sx0 = (double)(upper ? other : sum);
    op.sx1 = (double)(upper ? sum : other);
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const int o = __builtin_amdgcn_update_dpp(0, ps4[p], 0x140, 0xF, 0xF, true);
        op.c1[p] = (upper ? ps4[p] : o) * 128;
    }
    // lane i: chunk i / 16, half (i % 16) / 4, k-slots 4 * (i % 4) .. + 3
    uint8_t *at = area + g * 256u + (r >> 2) * 16u + (r & 3u) * 4u;
#pragma unroll
    for (int p = 0; p < 4; ++p) *reinterpret_cast<uint32_t *>(at + 64 * p) = dw[p];
}

// Chunk g of row r as the products want it (hdr: the superblock's first 16 bytes, ca / cb: the
// chunk's 32 code bytes).
struct q4k_one_weights {
    lev_i32x4 la, lb, ha, hb;   // B operands: low nibbles as q, high nibbles as 16 * (q - 8)
    int sc0, sc1;               // scales of sub-blocks 2g (x 16: the high sub-block's codes carry a 16) and 2g + 1
    double m0, m1, d, dmin;
};

__device__ __forceinline__ q4k_one_weights q4k_one_unpack(const lev_i32x4 hdr, const lev_i32x4 ca, const lev_i32x4 cb,
                                                          uint32_t g) {
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    q4k_one_weights W;
    // unpack_scale_min (lev-cpu/src/lib.rs:64-74), four sub-blocks a word; this lane wants sub-blocks
    // 2g and 2g + 1: bytes 2 * (g % 2) and + 1 of word g / 2
    const uint32_t S0 = (uint32_t)hdr[1], S1 = (uint32_t)hdr[2], S2 = (uint32_t)hdr[3];
    // (both words are formed and one is kept by a bit select: a conditional here becomes a branch)
    const uint32_t up = g >= 2u ? ~0u : 0u;
    const uint32_t sc_hi = (S2 & 0x0F0F0F0Fu) | ((S0 >> 2) & 0x30303030u), sc_lo = S0 & 0x3F3F3F3Fu;
    const uint32_t mn_hi = ((S2 >> 4) & 0x0F0F0F0Fu) | ((S1 >> 2) & 0x30303030u), mn_lo = S1 & 0x3F3F3F3Fu;
    const uint32_t scw = (sc_hi & up) | (sc_lo & ~up);
    const uint32_t mnw = (mn_hi & up) | (mn_lo & ~up);
    const uint32_t sh = 16u * (g & 1u);
    W.sc0 = (int)__builtin_amdgcn_ubfe(scw, sh, 8u) * 16;
    W.sc1 = (int)__builtin_amdgcn_ubfe(scw, sh + 8u, 8u);
    W.m0 = (double)__builtin_amdgcn_ubfe(mnw, sh, 8u);
    W.m1 = (double)__builtin_amdgcn_ubfe(mnw, sh + 8u, 8u);
    const u4 qa = __builtin_bit_cast(u4, ca), qb = __builtin_bit_cast(u4, cb);
    W.la = __builtin_bit_cast(lev_i32x4, qa & 0x0F0F0F0Fu);
    W.lb = __builtin_bit_cast(lev_i32x4, qb & 0x0F0F0F0Fu);
    W.ha = __builtin_bit_cast(lev_i32x4, (qa & 0xF0F0F0F0u) ^ 0x80808080u);
    W.hb = __builtin_bit_cast(lev_i32x4, (qb & 0xF0F0F0F0u) ^ 0x80808080u);
    W.d = (double)lev_f16_bits_to_f32((uint32_t)hdr[0] & 0xFFFFu);
    W.dmin = (double)lev_f16_bits_to_f32((uint32_t)hdr[0] >> 16);
    return W;
}

// Contribution of the chunk to the row's dot product with one column (a: the column's A operands,
// elements 16h .. 16h+15 of the lane group's 64, zeros outside the group's rows).
__device__ __forceinline__ double q4k_one_dot(const q4k_one_weights &W, const lev_i32x4 (&a)[4], const q4k_one_column &op) {
    lev_i32x4 d0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[0], W.la, lev_i32x4{0, 0, 0, 0}, 0, 0, 0);
    lev_i32x4 d1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[2], W.ha, lev_i32x4{0, 0, 0, 0}, 0, 0, 0);
    d0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[1], W.lb, d0, 0, 0, 0);
    d1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[3], W.hb, d1, 0, 0, 0);
    // |d0| < 2^16, |d1 + c1| < 2^20, scales below 2^10: every product and sum fits 32 bits
    int E[4];
#pragma unroll
    for (int p = 0; p < 4; ++p) E[p] = __mul24(d0[p], W.sc0) + __mul24(d1[p] + op.c1[p], W.sc1);
    // plane 3 is the highest digit (at most 2 in magnitude): E[3] * 256 + E[2] stays below 2^29
    const double hi = (double)(E[3] * 256 + E[2]);
    const double lo = fma((double)E[1], 256.0, (double)E[0]);
    const double dot = fma(hi, 65536.0, lo);                             // 16 * sum_j sc_j sum_k q_k X_k
    const double mins = fma(W.m1, op.sx1, W.m0 * op.sx0) * 16.0;
    return op.ps * fma(W.d, dot, -W.dmin * mins);
}

// wave -> (slot, superblock) as 4-bit entries of two 64-bit kernel arguments (no division in
// front of the first load).  NC: columns staged (1, 2 or 4; >= ncol): one column keeps its A
// operands in registers, several read them from the wave's planes at every product.
// NORM: RMSNorm (gain != nullptr) in front.
template <int NC, bool NORM>
__global__ void __launch_bounds__(kOneThreads)
q4_k_mfma_gemv_one(const uint8_t *__restrict__ w, const float *__restrict__ x, const float *__restrict__ gain,
                   float eps, float *__restrict__ y, uint32_t cols, uint32_t rows, uint32_t ncol, uint32_t wpr,
                   uint32_t slots, uint64_t slot_of_wave, uint64_t pos_of_wave, double rcols) {
    constexpr uint32_t kPart = q4k_one_part_bytes(NC), kNorm = q4k_one_norm_bytes(NC), kWave = q4k_one_wave_bytes(NC);
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const uint32_t slot = (uint32_t)(slot_of_wave >> (4u * wave)) & 15u;   // idle waves: slot >= slots
    const uint32_t sb = (uint32_t)(pos_of_wave >> (4u * wave)) & 15u;      // the wave's superblock column
    const uint32_t SB = cols >> 8;

    // the wave's activations first (short, mostly L2 hits; columns of the layout beyond ncol
    // repeat the last one and are never stored) ...
    lev_f32x4 v[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        const uint32_t cc = (uint32_t)c < ncol ? (uint32_t)c : ncol - 1u;
        v[c] = reinterpret_cast<const lev_f32x4 *>(x + (uint64_t)cc * cols)[64u * sb + lane];
    }
    lev_f32x4 gn;
    if (NORM) gn = reinterpret_cast<const lev_f32x4 *>(gain)[64u * sb + lane];
    // ... the first row group's weights right behind them
    const bool active = slot < slots;
    const uint64_t row_bytes = (uint64_t)SB * 144u;
    const uint32_t ngroups = (rows + 15u) >> 4;
    const uint32_t nrounds = (ngroups + slots - 1u) / slots;     // rounds of `slots` row groups
    const uint32_t lrow = lane >> 2;                             // fetch order: lane = 4 * row + chunk
    auto issue = [&](uint32_t round_block, uint32_t (&D)[9]) {
        uint32_t rg = round_block * slots + (active ? slot : 0u);
        rg = rg < ngroups ? rg : ngroups - 1u;
        uint32_t row = rg * 16u + lrow;
        row = row < rows ? row : rows - 1u;
        // lane 4 * row + c: dword c of the superblock's header and the 32 code bytes of chunk c
        // (a quad reads the row's 16 + 128 bytes)
        const uint8_t *p = w + (uint64_t)row * row_bytes + (uint64_t)sb * 144u;
        const uint32_t c = lane & 3u;
        typedef uint32_t u4 __attribute__((ext_vector_type(4)));
        D[0] = *reinterpret_cast<const uint32_t *>(p + 4u * c);
        const u4 a = *reinterpret_cast<const u4 *>(p + 16u + 32u * c);
        const u4 b = *reinterpret_cast<const u4 *>(p + 32u + 32u * c);
        D[1] = a.x; D[2] = a.y; D[3] = a.z; D[4] = a.w;
        D[5] = b.x; D[6] = b.y; D[7] = b.z; D[8] = b.w;
    };
    uint32_t D[9];
    uint32_t rb = blockIdx.x;
    if (NORM) {
        // A CU's memory pipeline is one queue: without this barrier the activations of the last
        // wave to start stand behind the weight requests of fifteen others, and every wave
        // waits for them at the sum of squares (1 us at 12288 x 4096).
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("s_barrier" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
    }
    issue(rb, D);

    // ---- everything the tail of a round needs, while the loads are on their way ----
    double *norm = reinterpret_cast<double *>(smem + kPart);
    uint8_t *area = smem + kPart + kNorm + (size_t)wave * kWave;
    uint8_t *zero = area + NC * kQ4mTaskArea;
    const uint32_t r = lane & 15u, q = lane >> 4;
    // byte offsets into the workgroup's LDS, not pointers (an address that has been through an
    // integer register is no longer known to be LDS)
    uint32_t pw = ((wave * 16u + lane) * NC) * 8u;
    // wave s < slots adds the wpr partial sums of slot s: lane (r, q) reads waves q, q + 4, q + 8, q + 12
    uint32_t pr = ((((wave < slots ? wave : 0u) * wpr + q) * 16u + r) * NC) * 8u;
    uint32_t k0 = q < wpr ? 1u : 0u, k1 = q + 4u < wpr ? 1u : 0u, k2 = q + 8u < wpr ? 1u : 0u,
             k3 = q + 12u < wpr ? 1u : 0u;
    uint32_t orow = (rb * slots + wave) * 16u + r;
    const uint32_t orow_step = gridDim.x * slots * 16u;
    const bool writer = wave < slots && q == 0u;
    uint32_t stores = writer && orow < rows ? 1u : 0u;
    uint64_t yp = reinterpret_cast<uint64_t>(y + orow);
    lev_pin(pw);
    lev_pin(pr);
    lev_pin(k0);
    lev_pin(k1);
    lev_pin(k2);
    lev_pin(k3);
    lev_pin(stores);
    lev_pin(yp);

    if (NORM) {
        // RMSNorm as the reference computes it (rmsnorm, rust/crates/lev-model/src/lib.rs:110-114):
        // mean square and 1/sqrt in f64, then (f32)(x * inv) * gain
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            double ss = (double)v[c].x * (double)v[c].x;
            ss = fma((double)v[c].y, (double)v[c].y, ss);
            ss = fma((double)v[c].z, (double)v[c].z, ss);
            ss = fma((double)v[c].w, (double)v[c].w, ss);
            ss = lev_group_sum_f64<64>(ss);                    // lane 63 holds the wave's sum
            if (lane == 63u) norm[c * kOneWaves + wave] = ss;
        }
        lev_barrier_lds();
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            // the waves of slot 0 cover the row once: lane k of every row of 16 lanes takes wave k's
            // sum, and the row adds them up (every lane ends with the total)
            const double mine = norm[c * kOneWaves + r];
            const double tot = lev_group_sum_f64<16>(r < wpr ? mine : 0.0);
            // 1/sqrt(mean + eps): the hardware estimate and two Newton steps (full f64 accuracy)
            const double a = fma(tot, rcols, (double)eps);
            double rs = __builtin_amdgcn_rsq(a);
            rs = rs * fma(-0.5 * a * rs, rs, 1.5);
            rs = rs * fma(-0.5 * a * rs, rs, 1.5);
#pragma unroll
            for (int k = 0; k < 4; ++k) v[c][k] = (float)((double)v[c][k] * rs) * gn[k];
        }
    }
    q4k_one_column op[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) q4k_one_stage(v[c], area + c * kQ4mTaskArea, active, op[c]);
    if (lane < kQ4mZeroBytes / 4u) reinterpret_cast<uint32_t *>(zero)[lane] = 0u;
    // the areas belong to this wave alone: LDS runs a wave's accesses in order, the fences only
    // keep the compiler from moving the reads above the writes
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const bool feeds = active && (r >> 2) == q;                // A row r belongs to lane group r / 4
    const uint8_t *ab = feeds ? area + q * 256u + (r & 3u) * 64u : zero;
    const uint32_t hs = feeds ? 16u : 0u, cs = feeds ? kQ4mTaskArea : 0u;
    lev_i32x4 a1[4];
    if (NC == 1) {
#pragma unroll
        for (int h = 0; h < 4; ++h) a1[h] = *reinterpret_cast<const lev_i32x4 *>(ab + h * hs);
    }
    // the operands are read back before the wait for the weights, not behind it
    __builtin_amdgcn_sched_barrier(0);

    // A round: the fetched dwords go to the lanes that multiply them, and the registers they came
    // in take the NEXT round's request at once (one round ahead and no more: with a second round
    // requested before the first is multiplied the same matrix streams in slower, 8.4 us against
    // 7.9 at 12288 x 4096; a workgroup walking adjacent rounds instead of rounds a grid apart: 8.1).
    // The request is unconditional (clamped): a branch around the loads would make the compiler
    // wait for them before the current group is multiplied.
    auto round = [&](uint32_t next_block) {
        // lane (r, q) <- lane 4r + q for the chunk, lanes 4r .. 4r + 3 for the header's four dwords
        lev_i32x4 hdr, ca, cb;
#pragma unroll
        for (int k = 0; k < 4; ++k) hdr[k] = __builtin_amdgcn_ds_bpermute((int)(16u * r + 4u * k), (int)D[0]);
        const int src = (int)((4u * r + q) * 4u);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            ca[k] = __builtin_amdgcn_ds_bpermute(src, (int)D[1 + k]);
            cb[k] = __builtin_amdgcn_ds_bpermute(src, (int)D[5 + k]);
        }
        // (the scheduling barriers keep the request where it is written: sunk below the products
        // it would no longer run ahead of anything)
        __builtin_amdgcn_sched_barrier(0);
        issue(next_block, D);
        __builtin_amdgcn_sched_barrier(0);
        const q4k_one_weights W = q4k_one_unpack(hdr, ca, cb, q);
        double val[NC];
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            if (NC == 1) {
                val[c] = q4k_one_dot(W, a1, op[c]);
            } else {
                lev_i32x4 a[4];
#pragma unroll
                for (int h = 0; h < 4; ++h) a[h] = *reinterpret_cast<const lev_i32x4 *>(ab + c * cs + h * hs);
                val[c] = q4k_one_dot(W, a, op[c]);
            }
            val[c] = lev_row_sum_f64(val[c]);
        }
        if (lane < 16u) {
#pragma unroll
            for (int c = 0; c < NC; ++c) *reinterpret_cast<double *>(smem + pw + 8 * c) = val[c];
        }
        lev_barrier_lds();
        if (wave < slots) {
            const double *pp = reinterpret_cast<const double *>(smem + pr);
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                const double p0 = pp[c], p1 = pp[64 * NC + c], p2 = pp[128 * NC + c], p3 = pp[192 * NC + c];
                double s = ((k0 ? p0 : 0.0) + (k1 ? p1 : 0.0)) + ((k2 ? p2 : 0.0) + (k3 ? p3 : 0.0));
                s = lev_row_sum_f64(s);
                if (stores && (uint32_t)c < ncol)
                    *reinterpret_cast<__attribute__((address_space(1))) float *>(yp + (uint64_t)c * rows * 4u) = (float)s;
            }
        }
        pw ^= kOneWaves * 16u * 8u * NC;                       // the other half of `part` next round
        pr ^= kOneWaves * 16u * 8u * NC;
        orow += orow_step;
        yp += (uint64_t)orow_step * 4u;
        stores = writer && orow < rows ? 1u : 0u;
    };
    while (true) {
        const uint32_t next = rb + gridDim.x;
        round(next < nrounds ? next : rb);
        if (next >= nrounds) break;
        rb = next;
    }
}

template <int NC, bool NORM>
hipError_t launch_one(lev_ctx *ctx, const uint8_t *w, const float *x, const float *gain, float eps, float *y,
                      uint32_t cols, uint32_t rows, uint32_t ncol) {
    const uint32_t wpr = cols >> 8, slots = (uint32_t)kOneWaves / wpr;
    const uint32_t ngroups = (rows + 15u) / 16u;
    const uint32_t nrounds = (ngroups + slots - 1u) / slots;
    uint64_t slot_of_wave, pos_of_wave;
    lev_wave_tables(wpr, &slot_of_wave, &pos_of_wave);
    constexpr size_t lds = q4k_one_lds(NC);
    if (lds > 48u * 1024u) {
        static bool configured = false;   // per instantiation: raise the dynamic LDS limit once
        if (!configured) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&q4_k_mfma_gemv_one<NC, NORM>),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return e;
            configured = true;
        }
    }
    const uint32_t cus = (uint32_t)ctx->num_cus;
    const uint32_t blocks = nrounds < cus ? nrounds : cus;
    hipLaunchKernelGGL((q4_k_mfma_gemv_one<NC, NORM>), dim3(blocks), dim3(kOneThreads), lds, ctx->stream, w, x, gain,
                       eps, y, cols, rows, ncol, wpr, slots, slot_of_wave, pos_of_wave, 1.0 / (double)cols);
    return hipGetLastError();
}

template <int NC>
hipError_t launch_one_nc(lev_ctx *ctx, const uint8_t *w, const float *x, const float *gain, float eps, float *y,
                         uint32_t cols, uint32_t rows, uint32_t ncol) {
    if (gain) return launch_one<NC, true>(ctx, w, x, gain, eps, y, cols, rows, ncol);
    return launch_one<NC, false>(ctx, w, x, gain, eps, y, cols, rows, ncol);
}

}  // namespace

// Shapes the kernel takes: one column, rows of one to sixteen whole superblocks.  (The kernel is
// written for NC columns, and two and four were measured at 12288 x 4096: 10.1 and 14.8 us against
// the 9.9 and 11.3 of q4_k_mfma_gemv, whose products carry four columns each.  Here a column costs
// its four products and some 75 vector instructions a round again, and with sixteen waves a CU
// the instruction count of a round, not the weight stream, then sets the time.)
bool lev_q4_k_mfma_one_usable(const uint8_t *w, const float *x, const float *gain, uint32_t in_dim, uint32_t ncol) {
    return ncol == 1u && in_dim % 256u == 0u && in_dim != 0u && in_dim <= 4096u &&
           (reinterpret_cast<uintptr_t>(w) & 3u) == 0u &&
           ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(gain)) & 15u) == 0u;
}

hipError_t lev_q4_k_mfma_one_launch(lev_ctx *ctx, const uint8_t *w, const float *x, const float *gain, float eps,
                                    float *y, uint32_t in_dim, uint32_t rows, uint32_t ncol) {
    return launch_one_nc<1>(ctx, w, x, gain, eps, y, in_dim, rows, ncol);
}

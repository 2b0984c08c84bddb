// RMSNorm + Q4_K multi-column GEMV on the integer matrix cores, for gfx950.
//
// Stands in for Builder::norm_quant + Builder::matvec with nb columns
// (rust/crates/lev-model/src/gpu.rs:295, 334-370; q4k.matvec,
// lev-forge/src/glsl.rs:157-281 and q8.rs:196-326): the weights are read once
// and applied to every column.
//
// One pass over W; at these sizes the vector ALU, not HBM, sets the time, so
// the formulation minimises instructions per weight.  Per superblock of 256
// weights of a row (w = d*sc_j*q - dmin*m_j, rust/crates/lev-cpu/src/lib.rs:111-154):
//
//   y += d * sum_j sc_j * (sum_k q_k x_k)  -  dmin * sum_j m_j * (sum_k x_k)
//
// Every sum is formed WITHOUT rounding:
//   * per superblock and column the activations become integers
//     X = rint(x * 2^(25-e)), 2^e the power of two above the superblock's largest
//     magnitude: |X| <= 2^25, a step of 2^-25 of that power of two (the top two
//     binades of f32 values are represented exactly).  X is written in four
//     balanced base-256 digits, X = ((b3*256 + b2)*256 + b1)*256 + b0 with every
//     b in [-128, 127] (|b3| <= 2): four int8 planes.
//   * v_mfma_i32_16x16x32_i8 per sub-block: the 16 A rows are 4 columns of x
//     times 4 digit planes, B is 16 weight rows x 32 codes (4-bit, unscaled).
//     The four planes of a column land in the four accumulator registers of one
//     lane, which multiplies them by the sub-block's 6-bit scale and adds them up
//     over the superblock in 32-bit integers (below 2^25 in magnitude per plane).
//   * once per superblock the planes are recombined in f64 (40-bit integers,
//     exact), d, dmin and the power of two are applied in f64, the partial sums of
//     a row are added in f64, and one rounding to f32 ends it.
// The result is the dot product of the dequantized row with the quantized
// activations, rounded once; the order of the additions does not show.
//
// lane (r, g) = (l % 16, l / 16) loads row r's 16-byte header and code bytes
// 8g..8g+7 of each 32-byte chunk (low nibbles: sub-block 2c, high: 2c+1); the
// output lane of weight row r is the lane that loaded its header.
//
// Workgroup = 16 waves, one per CU (the digit planes of four columns of 4096
// activations take 64 KB of LDS).  The waves of a workgroup share 16 weight rows,
// one superblock column each; their partial sums meet in LDS.
//
// Five to eight columns of at most sixteen superblocks: the planes are made once per launch
// by a small kernel in front (q4k_planes_kernel, below) instead of by every workgroup.
//
// A NaN or infinity in a column of x makes every output of that column NaN.
#include "lev_common.hpp"

#include <cstdlib>

namespace {

constexpr int kMThreads = 1024;
constexpr int kMWaves = kMThreads / LEV_WAVE;
constexpr uint32_t kNZeroBytes = 1024;   // what masked lanes of the narrow kernel read as their A operand

typedef int lev_i4 __attribute__((ext_vector_type(4)));
typedef uint32_t lev_u4 __attribute__((ext_vector_type(4)));
typedef uint32_t lev_u2 __attribute__((ext_vector_type(2)));
typedef double lev_d2 __attribute__((ext_vector_type(2)));

struct q4k_regs {
    lev_u4 hdr, a, b;
};

// Three 16-byte loads per lane: the header, and bytes [16*(g/2), +16) of chunk
// 2i + g%2 for i = 0, 1.  A wave's load covers 64 contiguous bytes per row.
__device__ __forceinline__ void q4k_issue(const uint8_t *__restrict__ w, uint64_t row_bytes, uint32_t row,
                                          uint32_t sb, uint32_t g, q4k_regs &R) {
    const uint8_t *p = w + (uint64_t)row * row_bytes + (uint64_t)sb * 144u;
    R.hdr = *reinterpret_cast<const lev_u4 *>(p);
    const uint8_t *q = p + 16u + 32u * (g & 1u) + 16u * (g >> 1);
    R.a = *reinterpret_cast<const lev_u4 *>(q);
    R.b = *reinterpret_cast<const lev_u4 *>(q + 64u);
}

// The MFMA wants bytes [8g, 8g+8) of every chunk in lane group g.  Lane groups g
// and g^1 (16 lanes apart) hold each other's second piece: the even group's upper
// half is the odd group's piece of chunk 2i, the odd group's lower half the even
// group's piece of chunk 2i+1.  One row swap per dword puts both in place:
// afterwards (x, y) is the lane's piece of chunk 2i and (z, w) of chunk 2i+1.
__device__ __forceinline__ void q4k_exchange(lev_u4 &v) {
    const auto s0 = __builtin_amdgcn_permlane16_swap(v.x, v.z, false, false);
    const auto s1 = __builtin_amdgcn_permlane16_swap(v.y, v.w, false, false);
    v.x = s0[0];
    v.z = s0[1];
    v.y = s1[0];
    v.w = s1[1];
}

// Byte offset of 16-byte unit u (= 8*kg + A row / 2) inside a sub-block's 512 bytes
// of digit planes.  The staging threads of one wave write units 8*kg + 2*(column % 4)
// of many sub-blocks at once; unswizzled, k-groups 0 and 2 and all sub-blocks would
// meet in the same banks.  Flipping bit 0 for the upper two k-groups and bit 1 for
// odd sub-blocks spreads eight consecutive lanes over eight bank groups, and is a
// permutation of the units inside a sub-block, so the MFMA's reads stay conflict-free.
__device__ __forceinline__ uint32_t q4k_unit(uint32_t u, uint32_t kg, uint32_t j) {
    return (u ^ (kg >> 1) ^ ((j & 1u) << 1)) * 16u;
}

// LDS, for SB superblocks and NL = 4*NX layout columns:
//   dig  [8*SB][NX][4 k-groups][16 A rows][8 bytes]   digit planes, A row = 4*(column % 4) + plane
//   sxd  [SB][NL][8] f64                               sum of X per sub-block
//   part [pb][wave][16 rows][NL] f64                   partial sums of a row group
//   psb  [SB][NL] f64                                  2^(e-25) per superblock
//   inv  [NL] f64, bad [NL] u32
//   run  [NL][8*SB] f64                                sums of squares (RMSNorm); in the digit area,
//                                                      which is written once they have been added up
template <int NX>
struct q4k_lds {
    static constexpr uint32_t NL = 4u * NX;
    static __host__ __device__ size_t dig_bytes(uint32_t subs) { return (size_t)subs * NX * 512u; }
    // pb: buffers for the partial sums (two save a barrier per row group)
    static __host__ __device__ size_t total(uint32_t subs, uint32_t pb) {
        return dig_bytes(subs) + (size_t)subs * NL * 8u + (size_t)pb * kMWaves * 16u * NL * 8u +
               (size_t)(subs >> 3) * NL * 8u + (size_t)NL * 12u;
    }
};

// ---------------------------------------------------------------------------
// The digit planes made ONCE per launch instead of once per workgroup.
//
// Turning a column of activations into digit planes costs a compute unit about a
// microsecond whoever does it, and in q4_k_mfma_gemv every workgroup does it for every
// column: at eight columns that is more than half of the kernel's instructions.  For five
// to eight columns of at most sixteen superblocks q4k_planes_kernel (one workgroup per
// column) writes the planes to device scratch in the order the matrix cores read them, and
// the workgroups of q4_k_mfma_gemv<NC, SHORT, true> load the planes of their wave's
// superblock column straight into registers: no staging, no digit area in LDS, no LDS read
// per product.  The numbers are the same integers, so the outputs are the same bits.
//
// Scratch, for NX groups of four layout columns and SB superblocks:
//   planes [SB][4 sub-block pairs][NX][64 lanes][16 B]   lane (r, g): A row r (4 * (column % 4) + plane,
//          plane 0 the highest digit), k-group g, of sub-blocks 2jp (low 8 bytes) and 2jp + 1 (high)
//   psb    [SB][4 * NX] f64                               2^(e-151) per superblock and column
//   bad    [4 * NX] u32                                   a NaN or infinity in the column
// The sum of X per sub-block (for the mins) is not stored: the matrix cores form
// sum_j m_j * sum_k digit directly, with the min of a sub-block in all of its B bytes.
// ---------------------------------------------------------------------------
constexpr int kPThreads = 512;   // one run of 8 activations per thread: in_dim <= 4096
__host__ __device__ constexpr size_t q4k_planes_bytes(uint32_t sb, uint32_t nx) { return (size_t)sb * nx * 4096u; }
__host__ __device__ constexpr size_t q4k_planes_total(uint32_t sb, uint32_t nx) {
    return q4k_planes_bytes(sb, nx) + (size_t)sb * 4u * nx * 8u + 4u * nx * 4u;
}

// grid (ncol), kPThreads threads; cols % 256 == 0, cols <= 8 * kPThreads; x and gain 16-byte aligned.
__global__ void __launch_bounds__(kPThreads)
q4k_planes_kernel(const float *__restrict__ x, const float *__restrict__ gain, float eps, uint8_t *__restrict__ scratch,
                  uint32_t cols, uint32_t nx, double rcols) {
    __shared__ double run[kPThreads / 4];
    __shared__ double s_inv;
    __shared__ uint32_t s_bad;
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t c = blockIdx.x, SB = cols >> 8, subs = cols >> 5, NL = 4u * nx;
    uint8_t *planes = scratch;
    double *psb = reinterpret_cast<double *>(scratch + q4k_planes_bytes(SB, nx));
    uint32_t *bad = reinterpret_cast<uint32_t *>(psb + (size_t)SB * NL);
    const bool real = tid < (cols >> 3);
    const uint32_t k8 = real ? tid : 0u;
    const lev_f32x4 *xp = reinterpret_cast<const lev_f32x4 *>(x + (uint64_t)c * cols) + 2u * k8;
    lev_f32x4 va = xp[0], vb = xp[1];
    if (tid == 0u) s_bad = 0u;
    if (gain) {
        const lev_f32x4 *gp = reinterpret_cast<const lev_f32x4 *>(gain) + 2u * k8;
        const lev_f32x4 ga = gp[0], gb = gp[1];
        // RMSNorm as the reference computes it (rmsnorm, rust/crates/lev-model/src/lib.rs:110-114):
        // mean square and 1/sqrt in f64, then (f32)(x * inv) * gain; the additions in the order of
        // q4_k_mfma_gemv (a sub-block's four runs, the sub-blocks lane by lane, the lanes)
        double ss = (double)va.x * (double)va.x;
        ss = fma((double)va.y, (double)va.y, ss); ss = fma((double)va.z, (double)va.z, ss);
        ss = fma((double)va.w, (double)va.w, ss); ss = fma((double)vb.x, (double)vb.x, ss);
        ss = fma((double)vb.y, (double)vb.y, ss); ss = fma((double)vb.z, (double)vb.z, ss);
        ss = fma((double)vb.w, (double)vb.w, ss);
        ss = lev_group_sum_f64<4>(ss);
        if (real && (k8 & 3u) == 3u) run[k8 >> 2] = ss;
        lev_barrier_lds();
        if (wave == 0u) {
            double tot = 0.0;
            for (uint32_t k = lane; k < subs; k += 64u) tot += run[k];
            tot = lev_group_sum_f64<64>(tot);
            const double a = fma(tot, rcols, (double)eps);
            double rs = __builtin_amdgcn_rsq(a);
            rs = rs * fma(-0.5 * a * rs, rs, 1.5);
            rs = rs * fma(-0.5 * a * rs, rs, 1.5);
            if (lane == 63u) s_inv = rs;
        }
        lev_barrier_lds();
        const double inv = s_inv;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            va[k] = (float)((double)va[k] * inv) * ga[k];
            vb[k] = (float)((double)vb[k] * inv) * gb[k];
        }
    } else {
        lev_barrier_lds();   // s_bad is zero before anybody raises it
    }
    const float v[8] = {va.x, va.y, va.z, va.w, vb.x, vb.y, vb.z, vb.w};
    uint32_t mb = 0u;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        const uint32_t bits = __float_as_uint(v[k]) & 0x7FFFFFFFu;
        mb = bits > mb ? bits : mb;
    }
    mb = lev_row16_max_u32(mb);
    {
        const uint32_t o = (uint32_t)__builtin_amdgcn_ds_swizzle((int)mb, 0x401F);   // lane ^ 16: the superblock's 32 runs
        mb = o > mb ? o : mb;
    }
    uint32_t ex = mb >> 23;
    if (real && ex == 255u) atomicOr(&s_bad, 1u);
    ex = ex < 25u ? 25u : (ex > 254u ? 254u : ex);
    const float scale = __uint_as_float((278u - ex) << 23);   // 2^(151-ex): |x*scale| < 2^25
    uint32_t dw[4][2];                                        // dw[3] = highest digit
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        uint32_t Y[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) Y[k] = ((uint32_t)(int)rintf(v[4 * h + k] * scale) + 0x00808080u) ^ 0x00808080u;
        const uint32_t t0 = __builtin_amdgcn_perm(Y[1], Y[0], 0x05010400u);
        const uint32_t t1 = __builtin_amdgcn_perm(Y[1], Y[0], 0x07030602u);
        const uint32_t t2 = __builtin_amdgcn_perm(Y[3], Y[2], 0x05010400u);
        const uint32_t t3 = __builtin_amdgcn_perm(Y[3], Y[2], 0x07030602u);
        dw[0][h] = __builtin_amdgcn_perm(t2, t0, 0x05040100u);
        dw[1][h] = __builtin_amdgcn_perm(t2, t0, 0x07060302u);
        dw[2][h] = __builtin_amdgcn_perm(t3, t1, 0x05040100u);
        dw[3][h] = __builtin_amdgcn_perm(t3, t1, 0x07060302u);
    }
    if (real) {
        const uint32_t j = k8 >> 2, kg = k8 & 3u;             // sub-block of the row, k-group
        const uint32_t sb = j >> 3, jp = (j & 7u) >> 1, half = j & 1u, q = c >> 2;
        uint8_t *at = planes + ((((size_t)sb * 4u + jp) * nx + q) * 64u + 16u * kg + 4u * (c & 3u)) * 16u + 8u * half;
#pragma unroll
        for (int p = 0; p < 4; ++p) *reinterpret_cast<lev_u2 *>(at + 16 * p) = lev_u2{dw[3 - p][0], dw[3 - p][1]};
        if ((k8 & 31u) == 31u) psb[sb * NL + c] = __hiloint2double((int)((ex + 872u) << 20), 0);   // 2^(ex-151)
    }
    lev_barrier_lds();
    if (tid == 0u) bad[c] = s_bad;
}

// NC: columns staged (1, 2, 4 or 8; >= ncol).  SHORT: no wave has more than
// three tasks (every decode-sized matrix); the kernel is then straight-line
// code, so the wait before each task covers exactly that task's loads and each
// task is multiplied while the next streams in.
// PLANES: the digit planes come from q4k_planes_kernel (`x` then points at its scratch; gain
// and eps are not used): SB <= 16, so a wave has one superblock column and keeps its A
// operands in registers; LDS holds the partial sums only.
template <int NC, bool SHORT, bool PLANES = false>
__global__ void __launch_bounds__(kMThreads)
q4_k_mfma_gemv(const uint8_t *__restrict__ w, const float *__restrict__ x,
               const float *__restrict__ gain, float eps, float *__restrict__ y, uint32_t cols,
               uint32_t rows, uint32_t ncol, uint32_t pb, double rcols) {
    constexpr int NX = NC > 4 ? 2 : 1;
    using L = q4k_lds<NX>;
    constexpr uint32_t NL = L::NL;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const uint32_t SB = cols >> 8, subs = PLANES ? 0u : cols >> 5;
    uint8_t *dig = smem;
    double *sxd = reinterpret_cast<double *>(smem + L::dig_bytes(subs));
    double *part = sxd + (size_t)subs * NL;
    double *psb = part + (size_t)pb * kMWaves * 16u * NL;
    double *s_inv = psb + (size_t)SB * NL;
    uint32_t *s_bad = reinterpret_cast<uint32_t *>(s_inv + NL);
    double *run = reinterpret_cast<double *>(smem);

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;

    // ---- geometry of the weight stream ----
    const uint32_t r = lane & 15u, g = lane >> 4;
    const uint64_t row_bytes = (uint64_t)SB * 144u;
    const uint32_t ngroups = (rows + 15u) >> 4;
    const uint32_t tpr = (SB + kMWaves - 1u) / kMWaves;    // tasks per row group and wave
    const uint32_t ntasks = ((ngroups - blockIdx.x + gridDim.x - 1u) / gridDim.x) * tpr;
    // A cursor walks the wave's tasks in order: row group rg (stride gridDim.x),
    // within it superblock wave + 16*t for t < tpr.  A task past the end (or
    // past the wave's last superblock) reads the first bytes of the matrix.
    struct cursor {
        uint32_t k, rg, t;
    };
    auto advance = [&](cursor &c) {
        ++c.k;
        if (++c.t == tpr) {
            c.t = 0;
            c.rg += gridDim.x;
        }
    };
    auto issue = [&](cursor &c, q4k_regs &W) {
        const uint32_t sbw = wave + kMWaves * c.t;
        const bool real = c.k < ntasks && sbw < SB;
        uint32_t row = c.rg * 16u + r;
        row = row < rows ? row : rows - 1u;
        q4k_issue(w, row_bytes, real ? row : 0u, real ? sbw : 0u, real ? g : 0u, W);
        advance(c);
    };
    cursor ci{0u, blockIdx.x, 0u}, cc{0u, blockIdx.x, 0u};
    q4k_regs W0, W1, W2;

    // ---- the planes of this wave's superblock column, from q4k_planes_kernel's scratch ----
    lev_i4 Areg[4][NX];      // [sub-block pair][group of four columns]: A of sub-blocks 2jp (x, y) and 2jp + 1 (z, w)
    double pwreg[NX];        // 2^(e-151) of column 4q + g
    if constexpr (PLANES) {
        const uint8_t *scratch = reinterpret_cast<const uint8_t *>(x);
        const uint32_t sbw = wave < SB ? wave : SB - 1u;
        const double *psb_g = reinterpret_cast<const double *>(scratch + q4k_planes_bytes(SB, NX));
#pragma unroll
        for (int jp = 0; jp < 4; ++jp)
#pragma unroll
            for (int q = 0; q < NX; ++q)
                Areg[jp][q] = *reinterpret_cast<const lev_i4 *>(
                    scratch + ((((size_t)sbw * 4u + (uint32_t)jp) * NX + (uint32_t)q) * 64u + lane) * 16u);
#pragma unroll
        for (int q = 0; q < NX; ++q) pwreg[q] = psb_g[sbw * NL + 4u * (uint32_t)q + g];
        if (tid < NL) s_bad[tid] = reinterpret_cast<const uint32_t *>(psb_g + (size_t)SB * NL)[tid];
        issue(ci, W0);
        if constexpr (!SHORT) {
            issue(ci, W1);
            issue(ci, W2);
        }
        lev_barrier_lds();
    }
    if constexpr (!PLANES) {
        // ---- stage the activations ----
        // A thread takes runs of 8 consecutive elements (the 8 k-slots one lane
        // feeds to one MFMA).  Slot q = tid + i*1024: the 32 runs of one superblock
        // of one column sit in 32 adjacent lanes (q % 32), superblocks of the NC
        // columns alternate (q / 32 % NC).  The loads are unconditional (clamped) so
        // that they are in flight together; whole passes beyond the data are skipped.
        constexpr int CH = 4;                                   // slots per thread: NC*cols/8 <= 4096
        constexpr uint32_t kLogNC = NC == 8 ? 3u : NC == 4 ? 2u : NC == 2 ? 1u : 0u;
        const uint32_t total_slots = (cols >> 3) * NC;
        auto slot_of = [&](uint32_t q, uint32_t &c, uint32_t &k8) {
            c = (q >> 5) & (NC - 1u);
            k8 = ((q >> (5u + kLogNC)) << 5) | (q & 31u);
            return q < total_slots && c < ncol;
        };
        lev_f32x4 va[CH], vb[CH];
        {
            lev_f32x4 ga[CH], gb[CH];
    #pragma unroll
            for (int i = 0; i < CH; ++i) {
                if ((uint32_t)i * kMThreads >= total_slots) break;   // workgroup-uniform
                uint32_t c, k8;
                if (!slot_of(tid + (uint32_t)i * kMThreads, c, k8)) c = 0u, k8 = 0u;
                const lev_f32x4 *xp = reinterpret_cast<const lev_f32x4 *>(x + (uint64_t)c * cols) + 2u * k8;
                va[i] = xp[0];
                vb[i] = xp[1];
                const lev_f32x4 *gp = reinterpret_cast<const lev_f32x4 *>(gain ? gain : x) + 2u * k8;
                ga[i] = gp[0];
                gb[i] = gp[1];
            }
            if (tid < NL) s_bad[tid] = 0u;
            // RMSNorm as the reference computes it (rmsnorm, rust/crates/lev-model/src/lib.rs:110-114):
            // mean square and 1/sqrt in f64, then (f32)(x * inv) * gain
            if (gain) {
    #pragma unroll
                for (int i = 0; i < CH; ++i) {
                    if ((uint32_t)i * kMThreads >= total_slots) break;
                    uint32_t c, k8;
                    const bool real = slot_of(tid + (uint32_t)i * kMThreads, c, k8);
                    const lev_f32x4 a = va[i], b = vb[i];
                    double ss = (double)a.x * (double)a.x;
                    ss = fma((double)a.y, (double)a.y, ss); ss = fma((double)a.z, (double)a.z, ss);
                    ss = fma((double)a.w, (double)a.w, ss); ss = fma((double)b.x, (double)b.x, ss);
                    ss = fma((double)b.y, (double)b.y, ss); ss = fma((double)b.z, (double)b.z, ss);
                    ss = fma((double)b.w, (double)b.w, ss);
                    ss = lev_group_sum_f64<4>(ss);   // the four runs of a sub-block sit in four adjacent lanes
                    if (real && (k8 & 3u) == 3u) run[c * subs + (k8 >> 2)] = ss;
                }
            }
            // every wave of the workgroup has its activations: a CU's memory pipeline is
            // one queue, and weight loads of early waves would hold up the activation
            // loads of late ones.  The first weights stream in while the digits are made.
            lev_barrier_lds();
            issue(ci, W0);
            if constexpr (!SHORT) {
                issue(ci, W1);
                issue(ci, W2);
            }
            if (gain) {
                // one wave per column adds the column's sums of squares
                if (wave < ncol) {
                    double ss = 0.0;
                    for (uint32_t k = lane; k < subs; k += 64u) ss += run[wave * subs + k];
                    ss = lev_group_sum_f64<64>(ss);
                    // 1/sqrt(mean + eps): the hardware estimate and two Newton steps (full f64 accuracy)
                    const double a = fma(ss, rcols, (double)eps);
                    double rs = __builtin_amdgcn_rsq(a);
                    rs = rs * fma(-0.5 * a * rs, rs, 1.5);
                    rs = rs * fma(-0.5 * a * rs, rs, 1.5);
                    if (lane == 63u) s_inv[wave] = rs;
                }
                lev_barrier_lds();   // the sums (in the digit area) are dead from here
    #pragma unroll
                for (int i = 0; i < CH; ++i) {
                    if ((uint32_t)i * kMThreads >= total_slots) break;
                    uint32_t c, k8;
                    const bool real = slot_of(tid + (uint32_t)i * kMThreads, c, k8);
                    const double inv = s_inv[real ? c : 0u];
    #pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        va[i][k] = (float)((double)va[i][k] * inv) * ga[i][k];
                        vb[i][k] = (float)((double)vb[i][k] * inv) * gb[i][k];
                    }
                }
            }
        }
    #pragma unroll
        for (int i = 0; i < CH; ++i) {
            if ((uint32_t)i * kMThreads >= total_slots) break;
            uint32_t c, k8;
            const bool real = slot_of(tid + (uint32_t)i * kMThreads, c, k8);
            const lev_f32x4 a = va[i], b = vb[i];
            const float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
            // largest magnitude of the superblock as an integer: NaN and infinity sort above every number
            uint32_t mb = 0u;
    #pragma unroll
            for (int k = 0; k < 8; ++k) {
                const uint32_t bits = __float_as_uint(v[k]) & 0x7FFFFFFFu;
                mb = bits > mb ? bits : mb;
            }
            mb = lev_row16_max_u32(mb);   // all 16 lanes of a row hold the row's maximum
            {
                const uint32_t o = (uint32_t)__builtin_amdgcn_ds_swizzle((int)mb, 0x401F);   // lane ^ 16
                mb = o > mb ? o : mb;
            }
            uint32_t ex = mb >> 23;                             // biased exponent: |x| < 2^(ex-126)
            if (real && ex == 255u) atomicOr(&s_bad[c], 1u);
            ex = ex < 25u ? 25u : (ex > 254u ? 254u : ex);      // keeps both powers of two normal numbers
            const float scale = __uint_as_float((278u - ex) << 23);   // 2^(151-ex): |x*scale| < 2^25
            int sum = 0, X[8];
    #pragma unroll
            for (int k = 0; k < 8; ++k) {
                X[k] = (int)rintf(v[k] * scale);
                sum += X[k];
            }
            // balanced base-256 digits: adding 0x80 to each of the low three bytes carries
            // into the next digit where a byte exceeds 127, and flipping bit 7 subtracts the
            // 0x80 again, so the bytes of (X + 0x808080) ^ 0x808080 read as int8 are the
            // digits.  A 4x4 byte transpose puts digit k of four neighbours into one dword.
            uint32_t dw[4][2];                                  // dw[3] = highest digit
    #pragma unroll
            for (int h = 0; h < 2; ++h) {
                uint32_t Y[4];
    #pragma unroll
                for (int k = 0; k < 4; ++k) Y[k] = ((uint32_t)X[4 * h + k] + 0x00808080u) ^ 0x00808080u;
                const uint32_t t0 = __builtin_amdgcn_perm(Y[1], Y[0], 0x05010400u);   // a0 b0 a1 b1
                const uint32_t t1 = __builtin_amdgcn_perm(Y[1], Y[0], 0x07030602u);   // a2 b2 a3 b3
                const uint32_t t2 = __builtin_amdgcn_perm(Y[3], Y[2], 0x05010400u);   // c0 d0 c1 d1
                const uint32_t t3 = __builtin_amdgcn_perm(Y[3], Y[2], 0x07030602u);   // c2 d2 c3 d3
                dw[0][h] = __builtin_amdgcn_perm(t2, t0, 0x05040100u);                // a0 b0 c0 d0
                dw[1][h] = __builtin_amdgcn_perm(t2, t0, 0x07060302u);
                dw[2][h] = __builtin_amdgcn_perm(t3, t1, 0x05040100u);
                dw[3][h] = __builtin_amdgcn_perm(t3, t1, 0x07060302u);
            }
            sum += __builtin_amdgcn_update_dpp(0, sum, 0xB1, 0xF, 0xF, true);   // 32 values of at most 2^25
            sum += __builtin_amdgcn_update_dpp(0, sum, 0x4E, 0xF, 0xF, true);
            if (real) {
                const uint32_t j = k8 >> 2, kg = k8 & 3u;       // sub-block, k-group
                // 16-byte unit u = 8*kg + (A row)/2 of the sub-block's 512 bytes, stored at q4k_unit(u, kg, j)
                uint8_t *blk = dig + ((size_t)j * NX + (c >> 2)) * 512u;
                const uint32_t u = 8u * kg + 2u * (c & 3u);
                *reinterpret_cast<lev_u4 *>(blk + q4k_unit(u, kg, j)) = lev_u4{dw[3][0], dw[3][1], dw[2][0], dw[2][1]};
                *reinterpret_cast<lev_u4 *>(blk + q4k_unit(u + 1u, kg, j)) = lev_u4{dw[1][0], dw[1][1], dw[0][0], dw[0][1]};
                if (kg == 3u) sxd[((j >> 3) * NL + c) * 8u + (j & 7u)] = (double)sum;
                if ((k8 & 31u) == 31u) psb[(j >> 3) * NL + c] = __hiloint2double((int)((ex + 872u) << 20), 0);   // 2^(ex-151)
            }
        }
        // columns of the layout beyond ncol hold no data: the lanes that read them
        // only feed outputs that are never stored
        lev_barrier_lds();

    }
    // ---- stream the weights ----
    double yacc[NX];
#pragma unroll
    for (int q = 0; q < NX; ++q) yacc[q] = 0.0;

    // One task: superblock (wave + 16*t) of the 16 rows of group rg.  After the
    // last task of a row group the waves' partial sums meet in LDS.
    uint32_t parity = 0;
    auto compute = [&](cursor &c, const q4k_regs &W) {
        const uint32_t rg = c.rg, t = c.t;
        const uint32_t sbw = wave + kMWaves * t;
        const bool live = sbw < SB;
        const uint32_t sb = live ? sbw : SB - 1u;
        // unpack_scale_min, lev-cpu/src/lib.rs:64-74: the eight scales and the eight mins as bytes
        const uint32_t S0 = W.hdr.y, S1 = W.hdr.z, S2 = W.hdr.w;
        const uint32_t sc_w[2] = {S0 & 0x3F3F3F3Fu, (S2 & 0x0F0F0F0Fu) | ((S0 >> 2) & 0x30303030u)};
        const uint32_t mn_w[2] = {S1 & 0x3F3F3F3Fu, ((S2 >> 4) & 0x0F0F0F0Fu) | ((S1 >> 2) & 0x30303030u)};
        int E[NX][4];
        double acc2[NX];
        lev_d2 SX[NX][4];
        double pw[NX];
        lev_i4 M[NX];            // PLANES: sum_j m_j * (sum of the sub-block's digits), per plane
#pragma unroll
        for (int q = 0; q < NX; ++q) {
            E[q][0] = E[q][1] = E[q][2] = E[q][3] = 0;
            acc2[q] = 0.0;
            M[q] = lev_i4{0, 0, 0, 0};
            if constexpr (PLANES) {
                pw[q] = pwreg[q];
            } else {
                const uint32_t m = sb * NL + 4u * q + g;
                pw[q] = psb[m];
#pragma unroll
                for (int h = 0; h < 4; ++h) SX[q][h] = *reinterpret_cast<const lev_d2 *>(sxd + m * 8u + 2u * h);
            }
        }
        // lane (r, g) reads A row r, k-group g: unit 8g + r/2, its low or high 8 bytes
        const uint8_t *ablk = dig + (size_t)sb * 8u * NX * 512u;
        const uint32_t aoff = q4k_unit(8u * g + (r >> 1), g, 0u) + 8u * (r & 1u);
        lev_u4 ca = W.a, cb = W.b;
        q4k_exchange(ca);
        q4k_exchange(cb);
        const lev_u2 chunk[4] = {lev_u2{ca.x, ca.y}, lev_u2{ca.z, ca.w}, lev_u2{cb.x, cb.y}, lev_u2{cb.z, cb.w}};
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int sc = (int)((sc_w[j >> 2] >> (8 * (j & 3))) & 0xFFu);
            const double mnd = (double)((mn_w[j >> 2] >> (8 * (j & 3))) & 0xFFu);
            lev_u2 wv = chunk[j >> 1];
            if (j & 1) wv >>= 4;
            wv &= 0x0F0F0F0Fu;
            const long B = __builtin_bit_cast(long, wv);
#pragma unroll
            for (int q = 0; q < NX; ++q) {
                long A;
                if constexpr (PLANES) {
                    const lev_i4 a4 = Areg[j >> 1][q];
                    A = __builtin_bit_cast(long, (j & 1) ? lev_u2{(uint32_t)a4.z, (uint32_t)a4.w} : lev_u2{(uint32_t)a4.x, (uint32_t)a4.y});
                } else {
                    A = *reinterpret_cast<const long *>(ablk + ((size_t)j * NX + q) * 512u + (aoff ^ (32u * (j & 1))));
                }
                const lev_i4 D = __builtin_amdgcn_mfma_i32_16x16x32_i8(A, B, lev_i4{0, 0, 0, 0}, 0, 0, 0);
                // |D| <= 32*15*128 < 2^16, sc < 2^6: eight of the products fit 32 bits with room
#pragma unroll
                for (int p = 0; p < 4; ++p) {
                    E[q][p] += __mul24(D[p], sc);
                    asm("" : "+v"(E[q][p]));   // one multiply-add per plane: keeps the sums from being regrouped
                }
                if constexpr (!PLANES) acc2[q] = fma(mnd, SX[q][j >> 1][j & 1], acc2[q]);
            }
            if constexpr (PLANES) {
                if (j & 1) {
                    // the mins of sub-blocks j - 1 and j in every B byte of their halves of a 64-deep product:
                    // the sum over the pair of m * (sum of the sub-block's digits), per plane (below 2^21 over
                    // the superblock)
                    const uint32_t mw = mn_w[j >> 2];
                    const uint32_t m0 = __builtin_amdgcn_perm(0u, mw, 0x01010101u * (uint32_t)((j - 1) & 3));
                    const uint32_t m1 = __builtin_amdgcn_perm(0u, mw, 0x01010101u * (uint32_t)(j & 3));
                    const lev_i4 Bm = __builtin_bit_cast(lev_i4, lev_u4{m0, m0, m1, m1});
#pragma unroll
                    for (int q = 0; q < NX; ++q)
                        M[q] = __builtin_amdgcn_mfma_i32_16x16x64_i8(Areg[j >> 1][q], Bm, M[q], 0, 0, 0);
                }
            }
        }
        // a task past the wave's last superblock contributes nothing
        const double d = live ? (double)lev_f16_bits_to_f32(W.hdr.x & 0xFFFFu) : 0.0;
        const double dmin = live ? (double)lev_f16_bits_to_f32(W.hdr.x >> 16) : 0.0;
#pragma unroll
        for (int q = 0; q < NX; ++q) {
            // plane 0 is the highest digit (at most 2 in magnitude); each plane is below 2^25
            const double hi = fma((double)E[q][0], 256.0, (double)E[q][1]);
            const double lo = fma((double)E[q][2], 256.0, (double)E[q][3]);
            const double dot = fma(hi, 65536.0, lo);
            if constexpr (PLANES) {
                const double mhi = fma((double)M[q][0], 256.0, (double)M[q][1]);
                const double mlo = fma((double)M[q][2], 256.0, (double)M[q][3]);
                acc2[q] = fma(mhi, 65536.0, mlo);
            }
            yacc[q] = fma(pw[q], fma(d, dot, -dmin * acc2[q]), yacc[q]);
        }

        if (t + 1u == tpr) {   // workgroup-uniform
            double *pp = part + parity * (kMWaves * 16u * NL);
            parity ^= pb - 1u;
#pragma unroll
            for (int q = 0; q < NX; ++q) {
                pp[(wave * 16u + r) * NL + 4u * q + g] = yacc[q];
                yacc[q] = 0.0;
            }
            lev_barrier_lds();
            if (tid < 16u * NL) {
                const uint32_t col = tid >> 4, rr = tid & 15u, row = rg * 16u + rr;
                double sum = 0.0;
#pragma unroll
                for (int kk = 0; kk < kMWaves; ++kk) sum += pp[((uint32_t)kk * 16u + rr) * NL + col];
                if (col < ncol && row < rows)
                    y[(uint64_t)col * rows + row] = s_bad[col] ? __builtin_nanf("") : (float)sum;
            }
            if (pb == 1u) lev_barrier_lds();   // the one buffer is written again by the next group
        }
        advance(c);
    };

    if constexpr (SHORT) {
        // A wave that issues a load while the CU's memory queue is full waits until the
        // queue drains: with all three tasks requested up front the waves sat in those
        // waits while the digits were still to be made, and multiplied nothing until
        // the last byte had arrived.  One task is requested before the digits, the
        // next two each just ahead of the multiply that precedes their use.
        issue(ci, W1);
        __builtin_amdgcn_sched_barrier(0);
        compute(cc, W0);
        __builtin_amdgcn_sched_barrier(0);
        issue(ci, W2);
        __builtin_amdgcn_sched_barrier(0);
        if (ntasks > 1u) compute(cc, W1);
        if (ntasks > 2u) compute(cc, W2);
        return;
    }
    // Three tasks in flight per wave.
    // The scheduling barriers keep a refill's loads behind the compute that
    // frees its registers: hoisted above it they would be younger than the
    // data the compute waits for, and the wait would cover them too.
    while (true) {
        compute(cc, W0);
        __builtin_amdgcn_sched_barrier(0);
        issue(ci, W0);
        __builtin_amdgcn_sched_barrier(0);
        if (cc.k >= ntasks) break;
        compute(cc, W1);
        __builtin_amdgcn_sched_barrier(0);
        issue(ci, W1);
        __builtin_amdgcn_sched_barrier(0);
        if (cc.k >= ntasks) break;
        compute(cc, W2);
        __builtin_amdgcn_sched_barrier(0);
        issue(ci, W2);
        __builtin_amdgcn_sched_barrier(0);
        if (cc.k >= ntasks) break;
    }
}

// One or two columns: the same sums with half the matrix-core products and half the
// multiply-adds.  v_mfma_i32_16x16x64_i8 takes 64 codes of 16 rows; lane group g
// (l / 16) supplies the 16 codes of ONE half sub-block -- exactly the 16 bytes it
// loaded (low or high nibbles), so nothing is exchanged between lanes -- and A row
// 4*gs + p holds digit plane p of the elements lane group gs supplies and zeros
// elsewhere: output row 4*gs + p is the plane sum over that half sub-block alone, in
// a lane of the group that holds the sub-block's scale.  (With four columns per MFMA,
// as above, three quarters of the lanes of a one-column launch multiply-add columns
// that do not exist.)  The digit planes take 4 bytes per element and column, so rows
// up to 32768 / NC wide are served.
//   dig  [NC][16*SB groups of 16][4 planes][16 bytes]
//   sx16 [NC][16*SB] i32                                sum of X per group of 16
//   part [pb][wave][16 rows][NC] f64, psb [NC][SB] f64, inv [NC] f64, bad [NC] u32
//   run  [NC][8*SB] f64 (RMSNorm), in the digit area
template <int NC>
struct q4k_narrow_lds {
    static __host__ __device__ size_t dig_bytes(uint32_t cols) { return (size_t)NC * cols * 4u; }
    static __host__ __device__ size_t total(uint32_t cols, uint32_t pb) {
        return dig_bytes(cols) + kNZeroBytes + (size_t)NC * (cols >> 4) * 4u +
               (size_t)pb * kMWaves * 16u * NC * 8u + (size_t)NC * (cols >> 8) * 8u + (size_t)NC * 12u + 8u;
    }
};

template <int NC, bool SHORT>
__global__ void __launch_bounds__(kMThreads)
q4_k_mfma_gemv_narrow(const uint8_t *__restrict__ w, const float *__restrict__ x,
               const float *__restrict__ gain, float eps, float *__restrict__ y, uint32_t cols,
               uint32_t rows, uint32_t ncol, uint32_t pb, double rcols) {
    using L = q4k_narrow_lds<NC>;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const uint32_t SB = cols >> 8, subs = cols >> 5;
    uint8_t *dig = smem;
    uint8_t *zero = smem + L::dig_bytes(cols);
    double *part = reinterpret_cast<double *>(zero + kNZeroBytes);
    double *psb = part + (size_t)pb * kMWaves * 16u * NC;
    double *s_inv = psb + (size_t)SB * NC;
    int32_t *sx16 = reinterpret_cast<int32_t *>(s_inv + NC);
    uint32_t *s_bad = reinterpret_cast<uint32_t *>(sx16 + (size_t)NC * (cols >> 4));
    double *run = reinterpret_cast<double *>(smem);

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;

    // ---- geometry of the weight stream ----
    const uint32_t r = lane & 15u, g = lane >> 4;
    const uint64_t row_bytes = (uint64_t)SB * 144u;
    const uint32_t ngroups = (rows + 15u) >> 4;
    const uint32_t tpr = (SB + kMWaves - 1u) / kMWaves;    // tasks per row group and wave
    const uint32_t ntasks = ((ngroups - blockIdx.x + gridDim.x - 1u) / gridDim.x) * tpr;
    // A cursor walks the wave's tasks in order: row group rg (stride gridDim.x),
    // within it superblock wave + 16*t for t < tpr.  A task past the end (or
    // past the wave's last superblock) reads the first bytes of the matrix.
    struct cursor {
        uint32_t k, rg, t;
    };
    auto advance = [&](cursor &c) {
        ++c.k;
        if (++c.t == tpr) {
            c.t = 0;
            c.rg += gridDim.x;
        }
    };
    auto issue = [&](cursor &c, q4k_regs &W) {
        const uint32_t sbw = wave + kMWaves * c.t;
        const bool real = c.k < ntasks && sbw < SB;
        uint32_t row = c.rg * 16u + r;
        row = row < rows ? row : rows - 1u;
        q4k_issue(w, row_bytes, real ? row : 0u, real ? sbw : 0u, real ? g : 0u, W);
        advance(c);
    };
    cursor ci{0u, blockIdx.x, 0u}, cc{0u, blockIdx.x, 0u};
    q4k_regs W0, W1, W2;

    // ---- stage the activations ----
    // A thread takes runs of 8 consecutive elements (the 8 k-slots one lane
    // feeds to one MFMA).  Slot q = tid + i*1024: the 32 runs of one superblock
    // of one column sit in 32 adjacent lanes (q % 32), superblocks of the NC
    // columns alternate (q / 32 % NC).  The loads are unconditional (clamped) so
    // that they are in flight together; whole passes beyond the data are skipped.
    constexpr int CH = 4;                                   // slots per thread: NC*cols/8 <= 4096
    constexpr uint32_t kLogNC = NC == 8 ? 3u : NC == 4 ? 2u : NC == 2 ? 1u : 0u;
    const uint32_t total_slots = (cols >> 3) * NC;
    auto slot_of = [&](uint32_t q, uint32_t &c, uint32_t &k8) {
        c = (q >> 5) & (NC - 1u);
        k8 = ((q >> (5u + kLogNC)) << 5) | (q & 31u);
        return q < total_slots && c < ncol;
    };
    lev_f32x4 va[CH], vb[CH];
    {
        lev_f32x4 ga[CH], gb[CH];
#pragma unroll
        for (int i = 0; i < CH; ++i) {
            if ((uint32_t)i * kMThreads >= total_slots) break;   // workgroup-uniform
            uint32_t c, k8;
            if (!slot_of(tid + (uint32_t)i * kMThreads, c, k8)) c = 0u, k8 = 0u;
            const lev_f32x4 *xp = reinterpret_cast<const lev_f32x4 *>(x + (uint64_t)c * cols) + 2u * k8;
            va[i] = xp[0];
            vb[i] = xp[1];
            const lev_f32x4 *gp = reinterpret_cast<const lev_f32x4 *>(gain ? gain : x) + 2u * k8;
            ga[i] = gp[0];
            gb[i] = gp[1];
        }
        if (tid < (uint32_t)NC) s_bad[tid] = 0u;
        if (tid < kNZeroBytes / 4u) reinterpret_cast<uint32_t *>(zero)[tid] = 0u;
        // RMSNorm as the reference computes it (rmsnorm, rust/crates/lev-model/src/lib.rs:110-114):
        // mean square and 1/sqrt in f64, then (f32)(x * inv) * gain
        if (gain) {
#pragma unroll
            for (int i = 0; i < CH; ++i) {
                if ((uint32_t)i * kMThreads >= total_slots) break;
                uint32_t c, k8;
                const bool real = slot_of(tid + (uint32_t)i * kMThreads, c, k8);
                const lev_f32x4 a = va[i], b = vb[i];
                double ss = (double)a.x * (double)a.x;
                ss = fma((double)a.y, (double)a.y, ss); ss = fma((double)a.z, (double)a.z, ss);
                ss = fma((double)a.w, (double)a.w, ss); ss = fma((double)b.x, (double)b.x, ss);
                ss = fma((double)b.y, (double)b.y, ss); ss = fma((double)b.z, (double)b.z, ss);
                ss = fma((double)b.w, (double)b.w, ss);
                ss = lev_group_sum_f64<4>(ss);   // the four runs of a sub-block sit in four adjacent lanes
                if (real && (k8 & 3u) == 3u) run[c * subs + (k8 >> 2)] = ss;
            }
        }
        // every wave of the workgroup has its activations: a CU's memory pipeline is
        // one queue, and weight loads of early waves would hold up the activation
        // loads of late ones.  The first weights stream in while the digits are made.
        lev_barrier_lds();
        issue(ci, W0);
        if constexpr (!SHORT) {
            issue(ci, W1);
            issue(ci, W2);
        }
        if (gain) {
            // one wave per column adds the column's sums of squares
            if (wave < ncol) {
                double ss = 0.0;
                for (uint32_t k = lane; k < subs; k += 64u) ss += run[wave * subs + k];
                ss = lev_group_sum_f64<64>(ss);
                // 1/sqrt(mean + eps): the hardware estimate and two Newton steps (full f64 accuracy)
                const double a = fma(ss, rcols, (double)eps);
                double rs = __builtin_amdgcn_rsq(a);
                rs = rs * fma(-0.5 * a * rs, rs, 1.5);
                rs = rs * fma(-0.5 * a * rs, rs, 1.5);
                if (lane == 63u) s_inv[wave] = rs;
            }
            lev_barrier_lds();   // the sums (in the digit area) are dead from here
#pragma unroll
            for (int i = 0; i < CH; ++i) {
                if ((uint32_t)i * kMThreads >= total_slots) break;
                uint32_t c, k8;
                const bool real = slot_of(tid + (uint32_t)i * kMThreads, c, k8);
                const double inv = s_inv[real ? c : 0u];
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    va[i][k] = (float)((double)va[i][k] * inv) * ga[i][k];
                    vb[i][k] = (float)((double)vb[i][k] * inv) * gb[i][k];
                }
            }
        }
    }
#pragma unroll
    for (int i = 0; i < CH; ++i) {
        if ((uint32_t)i * kMThreads >= total_slots) break;
        uint32_t c, k8;
        const bool real = slot_of(tid + (uint32_t)i * kMThreads, c, k8);
        const lev_f32x4 a = va[i], b = vb[i];
        const float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
        // largest magnitude of the superblock as an integer: NaN and infinity sort above every number
        uint32_t mb = 0u;
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const uint32_t bits = __float_as_uint(v[k]) & 0x7FFFFFFFu;
            mb = bits > mb ? bits : mb;
        }
        mb = lev_row16_max_u32(mb);   // all 16 lanes of a row hold the row's maximum
        {
            const uint32_t o = (uint32_t)__builtin_amdgcn_ds_swizzle((int)mb, 0x401F);   // lane ^ 16
            mb = o > mb ? o : mb;
        }
        uint32_t ex = mb >> 23;                             // biased exponent: |x| < 2^(ex-126)
        if (real && ex == 255u) atomicOr(&s_bad[c], 1u);
        ex = ex < 25u ? 25u : (ex > 254u ? 254u : ex);      // keeps both powers of two normal numbers
        const float scale = __uint_as_float((278u - ex) << 23);   // 2^(151-ex): |x*scale| < 2^25
        int sum = 0, X[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            X[k] = (int)rintf(v[k] * scale);
            sum += X[k];
        }
        // balanced base-256 digits: adding 0x80 to each of the low three bytes carries
        // into the next digit where a byte exceeds 127, and flipping bit 7 subtracts the
        // 0x80 again, so the bytes of (X + 0x808080) ^ 0x808080 read as int8 are the
        // digits.  A 4x4 byte transpose puts digit k of four neighbours into one dword.
        uint32_t dw[4][2];                                  // dw[3] = highest digit
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            uint32_t Y[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) Y[k] = ((uint32_t)X[4 * h + k] + 0x00808080u) ^ 0x00808080u;
            const uint32_t t0 = __builtin_amdgcn_perm(Y[1], Y[0], 0x05010400u);   // a0 b0 a1 b1
            const uint32_t t1 = __builtin_amdgcn_perm(Y[1], Y[0], 0x07030602u);   // a2 b2 a3 b3
            const uint32_t t2 = __builtin_amdgcn_perm(Y[3], Y[2], 0x05010400u);   // c0 d0 c1 d1
            const uint32_t t3 = __builtin_amdgcn_perm(Y[3], Y[2], 0x07030602u);   // c2 d2 c3 d3
            dw[0][h] = __builtin_amdgcn_perm(t2, t0, 0x05040100u);                // a0 b0 c0 d0
            dw[1][h] = __builtin_amdgcn_perm(t2, t0, 0x07060302u);
            dw[2][h] = __builtin_amdgcn_perm(t3, t1, 0x05040100u);
            dw[3][h] = __builtin_amdgcn_perm(t3, t1, 0x07060302u);
        }
        sum += __builtin_amdgcn_update_dpp(0, sum, 0xB1, 0xF, 0xF, true);   // the two runs of a group of 16
        if (real) {
            // group of 16 = k8 / 2, this run its low or high 8 bytes of every plane
            uint8_t *at = dig + (size_t)c * cols * 4u + (size_t)(k8 >> 1) * 64u + 8u * (k8 & 1u);
#pragma unroll
            for (int p = 0; p < 4; ++p) *reinterpret_cast<lev_u2 *>(at + 16 * p) = lev_u2{dw[p][0], dw[p][1]};
            if (k8 & 1u) sx16[c * (cols >> 4) + (k8 >> 1)] = sum;
            if ((k8 & 31u) == 31u) psb[c * SB + (k8 >> 5)] = __hiloint2double((int)((ex + 872u) << 20), 0);   // 2^(ex-151)
        }
    }
    // columns of the layout beyond ncol hold no data: the lanes that read them
    // only feed outputs that are never stored
    lev_barrier_lds();

    // ---- stream the weights ----
    double yacc[NC];
#pragma unroll
    for (int q = 0; q < NC; ++q) yacc[q] = 0.0;
    // lane (r, g): weight row r; its loads a and b are bytes [16*(g/2), +16) of chunks g%2 and
    // 2 + g%2, i.e. for load i and nibble nb the half g/2 of sub-block 2*(2i + g%2) + nb
    const uint32_t gh = g >> 1, gl = g & 1u;
    const bool feeds = (r >> 2) == g;                       // this lane's A row belongs to its own lane group
    const uint32_t a_lane = (4u * gl + gh) * 64u + 16u * (r & 3u);   // + (8i + 2nb) groups of 64 bytes

    // One task: superblock (wave + 16*t) of the 16 rows of group rg.  After the
    // last task of a row group the waves' partial sums meet in LDS.
    uint32_t parity = 0;
    auto compute = [&](cursor &c, const q4k_regs &W) {
        const uint32_t rg = c.rg, t = c.t;
        const uint32_t sbw = wave + kMWaves * t;
        const bool live = sbw < SB;
        const uint32_t sb = live ? sbw : SB - 1u;
        // unpack_scale_min, lev-cpu/src/lib.rs:64-74: the eight scales and the eight mins as bytes
        const uint32_t S0 = W.hdr.y, S1 = W.hdr.z, S2 = W.hdr.w;
        const uint32_t sc_w[2] = {S0 & 0x3F3F3F3Fu, (S2 & 0x0F0F0F0Fu) | ((S0 >> 2) & 0x30303030u)};
        const uint32_t mn_w[2] = {S1 & 0x3F3F3F3Fu, ((S2 >> 4) & 0x0F0F0F0Fu) | ((S1 >> 2) & 0x30303030u)};
        // sub-block j = 4i + 2*gl + nb: byte 2*gl + nb of word i
        int sc[2][2];
        double mnd[2][2];
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) {
                sc[i][nb] = (int)__builtin_amdgcn_ubfe(sc_w[i], 16u * gl + 8u * (uint32_t)nb, 8u);
                mnd[i][nb] = (double)__builtin_amdgcn_ubfe(mn_w[i], 16u * gl + 8u * (uint32_t)nb, 8u);
            }
        // B operands: the 16 code bytes as loaded, low or high nibbles
        lev_i4 B[2][2];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const lev_u4 v = i ? W.b : W.a;
            B[i][0] = __builtin_bit_cast(lev_i4, v & 0x0F0F0F0Fu);
            B[i][1] = __builtin_bit_cast(lev_i4, (v >> 4) & 0x0F0F0F0Fu);
        }
        // a task past the wave's last superblock contributes nothing
        const double d = live ? (double)lev_f16_bits_to_f32(W.hdr.x & 0xFFFFu) : 0.0;
        const double dmin = live ? (double)lev_f16_bits_to_f32(W.hdr.x >> 16) : 0.0;
        const uint32_t goff = 16u * sb + 4u * gl + gh;        // group of 16 of (i, nb) = (0, 0); + 8i + 2nb
#pragma unroll
        for (int q = 0; q < NC; ++q) {
            const uint8_t *ab = feeds ? dig + (size_t)q * cols * 4u + (size_t)sb * 1024u + a_lane : zero;
            const int32_t *sxp = sx16 + (size_t)q * (cols >> 4) + goff;
            int E[4] = {0, 0, 0, 0};
            double acc2 = 0.0;
#pragma unroll
            for (int i = 0; i < 2; ++i) {
#pragma unroll
                for (int nb = 0; nb < 2; ++nb) {
                    const lev_i4 A = *reinterpret_cast<const lev_i4 *>(ab + (8 * i + 2 * nb) * 64);
                    const lev_i4 D = __builtin_amdgcn_mfma_i32_16x16x64_i8(A, B[i][nb], lev_i4{0, 0, 0, 0}, 0, 0, 0);
                    // |D| <= 16*15*128 < 2^15, sc < 2^6: the four products per plane fit 32 bits with room
#pragma unroll
                    for (int p = 0; p < 4; ++p) {
                        E[p] += __mul24(D[p], sc[i][nb]);
                        asm("" : "+v"(E[p]));   // one multiply-add per plane: keeps the sums from being regrouped
                    }
                    acc2 = fma(mnd[i][nb], (double)sxp[8 * i + 2 * nb], acc2);
                }
            }
            // plane 3 is the highest digit (at most 2 in magnitude)
            const double hi = fma((double)E[3], 256.0, (double)E[2]);
            const double lo = fma((double)E[1], 256.0, (double)E[0]);
            const double dot = fma(hi, 65536.0, lo);
            yacc[q] = fma(psb[q * SB + sb], fma(d, dot, -dmin * acc2), yacc[q]);
        }

        if (t + 1u == tpr) {   // workgroup-uniform
            double *pp = part + parity * (kMWaves * 16u * NC);
            parity ^= pb - 1u;
#pragma unroll
            for (int q = 0; q < NC; ++q) {
                // the four lane groups hold the four quarters of the row's share
                double s = yacc[q];
                s += __shfl_xor(s, 16);
                s += __shfl_xor(s, 32);
                if (g == 0u) pp[(wave * 16u + r) * NC + q] = s;
                yacc[q] = 0.0;
            }
            lev_barrier_lds();
            if (tid < 16u * NC) {
                const uint32_t col = tid >> 4, rr = tid & 15u, row = rg * 16u + rr;
                double sum = 0.0;
#pragma unroll
                for (int kk = 0; kk < kMWaves; ++kk) sum += pp[((uint32_t)kk * 16u + rr) * NC + col];
                if (col < ncol && row < rows)
                    y[(uint64_t)col * rows + row] = s_bad[col] ? __builtin_nanf("") : (float)sum;
            }
            if (pb == 1u) lev_barrier_lds();   // the one buffer is written again by the next group
        }
        advance(c);
    };

    if constexpr (SHORT) {
        // A wave that issues a load while the CU's memory queue is full waits until the
        // queue drains: with all three tasks requested up front the waves sat in those
        // waits while the digits were still to be made, and multiplied nothing until
        // the last byte had arrived.  One task is requested before the digits, the
        // next two each just ahead of the multiply that precedes their use.
        issue(ci, W1);
        __builtin_amdgcn_sched_barrier(0);
        compute(cc, W0);
        __builtin_amdgcn_sched_barrier(0);
        issue(ci, W2);
        __builtin_amdgcn_sched_barrier(0);
        if (ntasks > 1u) compute(cc, W1);
        if (ntasks > 2u) compute(cc, W2);
        return;
    }
    // Three tasks in flight per wave.
    // The scheduling barriers keep a refill's loads behind the compute that
    // frees its registers: hoisted above it they would be younger than the
    // data the compute waits for, and the wait would cover them too.
    while (true) {
        compute(cc, W0);
        __builtin_amdgcn_sched_barrier(0);
        issue(ci, W0);
        __builtin_amdgcn_sched_barrier(0);
        if (cc.k >= ntasks) break;
        compute(cc, W1);
        __builtin_amdgcn_sched_barrier(0);
        issue(ci, W1);
        __builtin_amdgcn_sched_barrier(0);
        if (cc.k >= ntasks) break;
        compute(cc, W2);
        __builtin_amdgcn_sched_barrier(0);
        issue(ci, W2);
        __builtin_amdgcn_sched_barrier(0);
        if (cc.k >= ntasks) break;
    }
}

size_t q4k_mfma_lds_bytes(uint32_t cols, uint32_t nc, uint32_t pb) {
    return nc > 4u ? q4k_lds<2>::total(cols >> 5, pb) : q4k_lds<1>::total(cols >> 5, pb);
}

size_t q4k_lds_limit(const lev_ctx *ctx) {
    return ctx->props.sharedMemPerBlockOptin > ctx->props.sharedMemPerBlock ? ctx->props.sharedMemPerBlockOptin
                                                                            : ctx->props.sharedMemPerBlock;
}

template <int NC, bool SHORT>
hipError_t launch_mfma_variant(lev_ctx *ctx, const uint8_t *w, const float *x, const float *gain, float eps,
                       float *y, uint32_t cols, uint32_t rows, uint32_t ncol) {
    const uint32_t pb = q4k_mfma_lds_bytes(cols, NC, 2u) <= q4k_lds_limit(ctx) ? 2u : 1u;
    const size_t lds = q4k_mfma_lds_bytes(cols, NC, pb);
    static size_t configured = 0;   // per instantiation: raise the dynamic LDS limit once per size
    if (lds > 48 * 1024 && lds > configured) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&q4_k_mfma_gemv<NC, SHORT>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        configured = lds;
    }
    uint32_t groups = (rows + 15u) / 16u;
    uint32_t blocks = groups < (uint32_t)ctx->num_cus ? groups : (uint32_t)ctx->num_cus;
    hipLaunchKernelGGL((q4_k_mfma_gemv<NC, SHORT>), dim3(blocks), dim3(kMThreads), lds, ctx->stream, w,
                       x, gain, eps, y, cols, rows, ncol, pb, 1.0 / (double)cols);
    return hipGetLastError();
}

template <int NC>
hipError_t launch_mfma(lev_ctx *ctx, const uint8_t *w, const float *x, const float *gain, float eps,
                       float *y, uint32_t cols, uint32_t rows, uint32_t ncol) {
    const uint32_t groups = (rows + 15u) / 16u;
    const uint32_t blocks = groups < (uint32_t)ctx->num_cus ? groups : (uint32_t)ctx->num_cus;
    const uint32_t tpr = ((cols >> 8) + kMWaves - 1u) / kMWaves;
    const uint32_t most = ((groups + blocks - 1u) / blocks) * tpr;   // tasks of the busiest wave
    if (most <= 3u) return launch_mfma_variant<NC, true>(ctx, w, x, gain, eps, y, cols, rows, ncol);
    return launch_mfma_variant<NC, false>(ctx, w, x, gain, eps, y, cols, rows, ncol);
}

// Five to eight columns of at most sixteen superblocks: the planes once per launch (q4k_planes_kernel), then the
// products.  Returns hipErrorOutOfMemory when the scratch cannot be had (a program is being recorded and the
// context's scratch is still too small): the caller then takes the kernel that stages for itself (same bits).
template <int NC, bool SHORT>
hipError_t launch_planes_variant(lev_ctx *ctx, const uint8_t *w, const uint8_t *scratch, float *y, uint32_t cols,
                                 uint32_t rows, uint32_t ncol) {
    constexpr uint32_t NL = NC > 4 ? 8u : 4u, pb = 2u;
    const size_t lds = (size_t)pb * kMWaves * 16u * NL * 8u + (size_t)(cols >> 8) * NL * 8u + (size_t)NL * 12u;   // 34 KB
    const uint32_t groups = (rows + 15u) / 16u;
    const uint32_t blocks = groups < (uint32_t)ctx->num_cus ? groups : (uint32_t)ctx->num_cus;
    hipLaunchKernelGGL((q4_k_mfma_gemv<NC, SHORT, true>), dim3(blocks), dim3(kMThreads), lds, ctx->stream, w,
                       reinterpret_cast<const float *>(scratch), static_cast<const float *>(nullptr), 0.f, y, cols,
                       rows, ncol, pb, 0.0);
    return hipGetLastError();
}

// From how many columns the planes are made in front (LEV_Q4K_PLANES: 0 never, 3..8 from that many; built-in 5).
uint32_t q4k_planes_min_cols() {
    static const uint32_t v = [] {
        const char *e = getenv("LEV_Q4K_PLANES");
        const int n = e ? atoi(e) : 5;
        return e && e[0] == '0' ? 0xFFFFFFFFu : (uint32_t)(n < 3 ? 3 : n > 8 ? 8 : n);
    }();
    return v;
}

bool q4k_planes_serves(uint32_t cols, uint32_t ncol) {
    return ncol >= q4k_planes_min_cols() && ncol <= 8u && cols % 256u == 0u && cols != 0u && cols <= 8u * kPThreads &&
           (cols >> 8) <= (uint32_t)kMWaves;
}

hipError_t launch_planes(lev_ctx *ctx, const uint8_t *w, const float *x, const float *gain, float eps, float *y,
                         uint32_t cols, uint32_t rows, uint32_t ncol) {
    const uint32_t SB = cols >> 8, nx = ncol > 4u ? 2u : 1u;
    uint8_t *scratch = static_cast<uint8_t *>(lev_scratch(ctx, q4k_planes_total(SB, nx)));
    if (!scratch) return hipErrorOutOfMemory;
    hipLaunchKernelGGL(q4k_planes_kernel, dim3(ncol), dim3(kPThreads), 0, ctx->stream, x, gain, eps, scratch, cols, nx,
                       1.0 / (double)cols);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    const uint32_t groups = (rows + 15u) / 16u;
    const uint32_t blocks = groups < (uint32_t)ctx->num_cus ? groups : (uint32_t)ctx->num_cus;
    const bool few = (groups + blocks - 1u) / blocks <= 3u;
    if (nx == 2u)
        return few ? launch_planes_variant<8, true>(ctx, w, scratch, y, cols, rows, ncol)
                   : launch_planes_variant<8, false>(ctx, w, scratch, y, cols, rows, ncol);
    return few ? launch_planes_variant<4, true>(ctx, w, scratch, y, cols, rows, ncol)
               : launch_planes_variant<4, false>(ctx, w, scratch, y, cols, rows, ncol);
}

size_t q4k_narrow_lds_bytes(uint32_t cols, uint32_t nc, uint32_t pb) {
    return nc > 1u ? q4k_narrow_lds<2>::total(cols, pb) : q4k_narrow_lds<1>::total(cols, pb);
}

template <int NC, bool SHORT>
hipError_t launch_narrow_variant(lev_ctx *ctx, const uint8_t *w, const float *x, const float *gain, float eps,
                                 float *y, uint32_t cols, uint32_t rows, uint32_t ncol) {
    const uint32_t pb = q4k_narrow_lds_bytes(cols, NC, 2u) <= q4k_lds_limit(ctx) ? 2u : 1u;
    const size_t lds = q4k_narrow_lds_bytes(cols, NC, pb);
    static size_t configured = 0;   // per instantiation: raise the dynamic LDS limit once per size
    if (lds > 48 * 1024 && lds > configured) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&q4_k_mfma_gemv_narrow<NC, SHORT>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        configured = lds;
    }
    const uint32_t groups = (rows + 15u) / 16u;
    const uint32_t blocks = groups < (uint32_t)ctx->num_cus ? groups : (uint32_t)ctx->num_cus;
    hipLaunchKernelGGL((q4_k_mfma_gemv_narrow<NC, SHORT>), dim3(blocks), dim3(kMThreads), lds, ctx->stream, w,
                       x, gain, eps, y, cols, rows, ncol, pb, 1.0 / (double)cols);
    return hipGetLastError();
}

template <int NC>
hipError_t launch_narrow(lev_ctx *ctx, const uint8_t *w, const float *x, const float *gain, float eps,
                         float *y, uint32_t cols, uint32_t rows, uint32_t ncol) {
    const uint32_t groups = (rows + 15u) / 16u;
    const uint32_t blocks = groups < (uint32_t)ctx->num_cus ? groups : (uint32_t)ctx->num_cus;
    const uint32_t tpr = ((cols >> 8) + kMWaves - 1u) / kMWaves;
    const uint32_t most = ((groups + blocks - 1u) / blocks) * tpr;   // tasks of the busiest wave
    if (most <= 3u) return launch_narrow_variant<NC, true>(ctx, w, x, gain, eps, y, cols, rows, ncol);
    return launch_narrow_variant<NC, false>(ctx, w, x, gain, eps, y, cols, rows, ncol);
}

}  // namespace

// Columns one launch of the MFMA kernel can take for this in_dim (0: not usable).
uint32_t lev_q4_k_mfma_cols(const lev_ctx *ctx, uint32_t in_dim) {
    if (in_dim % 256u != 0u || in_dim == 0u) return 0;
    uint32_t nc = 8;
    const size_t limit = q4k_lds_limit(ctx);
    while (nc >= 1u && ((uint64_t)nc * in_dim > 32768u || q4k_mfma_lds_bytes(in_dim, nc, 1u) > limit))
        nc >>= 1;
    return nc;
}

// Columns the one- and two-column kernel can take for this in_dim (0: not usable).
uint32_t lev_q4_k_mfma_narrow_cols(const lev_ctx *ctx, uint32_t in_dim) {
    static const bool off = [] {
        const char *e = getenv("LEV_Q4K_NARROW");   // LEV_Q4K_NARROW=0: four columns per product, for comparison
        return e && e[0] == '0';
    }();
    if (off || in_dim % 256u != 0u || in_dim == 0u) return 0;
    const size_t limit = q4k_lds_limit(ctx);
    for (uint32_t nc = 2; nc >= 1u; --nc)
        if ((uint64_t)nc * in_dim <= 32768u && q4k_narrow_lds_bytes(in_dim, nc, 1u) <= limit) return nc;
    return 0;
}

bool lev_q4_k_mfma_one_usable(const uint8_t *w, const float *x, const float *gain, uint32_t in_dim, uint32_t ncol);
hipError_t lev_q4_k_mfma_one_launch(lev_ctx *ctx, const uint8_t *w, const float *x, const float *gain, float eps,
                                    float *y, uint32_t in_dim, uint32_t rows, uint32_t ncol);

// ncol <= lev_q4_k_mfma_narrow_cols(ctx, in_dim) (the narrow kernel) or
// ncol <= lev_q4_k_mfma_cols(ctx, in_dim); w 16-byte aligned.
hipError_t lev_q4_k_mfma_gemv_launch(lev_ctx *ctx, const uint8_t *w, const float *x, const float *gain,
                                     float eps, float *y, uint32_t in_dim, uint32_t rows,
                                     uint32_t ncol) {
    // one column of at most sixteen superblocks: a wave per superblock column (q4_k_mfma_gemv_one.hip)
    static const bool one_off = [] {
        const char *e = getenv("LEV_Q4K_ONE");   // LEV_Q4K_ONE=0: the narrow kernel at one column too, for comparison
        return e && e[0] == '0';
    }();
    if (!one_off && lev_q4_k_mfma_one_usable(w, x, gain, in_dim, ncol))
        return lev_q4_k_mfma_one_launch(ctx, w, x, gain, eps, y, in_dim, rows, ncol);
    // one column of a longer row: the narrow kernel (9.1 us against 9.7 at 12288 x 4096); two columns: only where the
    // four-column kernel's planes do not fit (it is the faster of the two there: 9.9 against 10.8 us)
    if (ncol <= lev_q4_k_mfma_narrow_cols(ctx, in_dim) && (ncol == 1u || lev_q4_k_mfma_cols(ctx, in_dim) < ncol)) {
        if (ncol > 1) return launch_narrow<2>(ctx, w, x, gain, eps, y, in_dim, rows, ncol);
        return launch_narrow<1>(ctx, w, x, gain, eps, y, in_dim, rows, ncol);
    }
    if (q4k_planes_serves(in_dim, ncol)) {
        const hipError_t e = launch_planes(ctx, w, x, gain, eps, y, in_dim, rows, ncol);
        if (e != hipErrorOutOfMemory) return e;
    }
    if (ncol > 4) return launch_mfma<8>(ctx, w, x, gain, eps, y, in_dim, rows, ncol);
    if (ncol > 2) return launch_mfma<4>(ctx, w, x, gain, eps, y, in_dim, rows, ncol);
    if (ncol > 1) return launch_mfma<2>(ctx, w, x, gain, eps, y, in_dim, rows, ncol);
    return launch_mfma<1>(ctx, w, x, gain, eps, y, in_dim, rows, ncol);
}

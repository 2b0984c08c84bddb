// RMSNorm + Q4_K multi-column GEMV on the matrix cores, for gfx950.
//
// Stands in for Builder::norm_quant + Builder::matvec with nb columns
// (rust/crates/lev-model/src/gpu.rs:295, 334-370; q4k.matvec,
// lev-forge/src/glsl.rs:157-281 and q8.rs:196-326): the weights are read once
// and applied to every column.
//
// Still HBM-bound (one pass over W); the matrix cores only take the multiplies
// off the vector ALU, which a plain FMA kernel saturates from three columns
// up.  Formulation, per superblock of 256 weights of a row
// (w = d*sc_j*q - dmin*m_j, rust/crates/lev-cpu/src/lib.rs:111-154):
//
//   y += d * sum_k (sc*q)_k * x_k  -  dmin * sum_j m_j * S_j,   S_j = sum of x over sub-block j
//
//   * (sc*q) <= 63*15 = 945 is formed with one integer multiply on two 16-bit
//     lanes at a time and IS the fp16 subnormal (sc*q)*2^-24 bit pattern: an
//     exact B operand with no conversion.  m_j (<= 63) likewise.
//   * x is split once per workgroup into fp16 high + low halves (after a
//     power-of-two column scale so that nothing overflows or underflows):
//     x = hi + lo to 2^-25 of the column maximum, products are exact in the
//     f32 accumulator, so the result matches an f32 FMA chain to rounding.
//   * v_mfma_f32_16x16x32_f16: A = x (16 "rows" = columns of x, up to 8 used),
//     B = 16 weight rows x 32 weights.  The output lane of weight row n is the
//     lane that loaded row n's superblock header, so d and dmin are applied
//     without any exchange.
//   * lane (r, g) = (l % 16, l / 16) loads 16-byte pieces g and g + 4 of row
//     r's 128 code bytes (a wave's load covers 64 contiguous bytes per row)
//     and the row's 16-byte header.  The 32 weights of a piece (16 low
//     nibbles, 16 high nibbles) fill the lane's k-slots of four MFMAs; the
//     activations sit in LDS already permuted into that order.
//
// Workgroup = 16 waves, one per CU (the staged activations take up to 128 KB
// of LDS).  The waves of a workgroup share 16 weight rows, one superblock
// column each; their partial sums meet in LDS and are added in wave order.
#include "lev_common.hpp"

namespace {

constexpr int kMThreads = 1024;
constexpr int kMWaves = kMThreads / LEV_WAVE;

typedef _Float16 lev_h8 __attribute__((ext_vector_type(8)));
typedef _Float16 lev_h4 __attribute__((ext_vector_type(4)));
typedef uint32_t lev_u4 __attribute__((ext_vector_type(4)));
typedef uint32_t lev_u2 __attribute__((ext_vector_type(2)));

// position of code byte b (0..3) of a dword among the four 16-bit k-slots that
// the dword's low (or high) nibbles produce: (w & 0x000F000F) holds bytes 0, 2
// and ((w >> 8) & 0x000F000F) bytes 1, 3.
__device__ __forceinline__ uint32_t kslot_of_byte(uint32_t b) { return ((b & 1u) << 1) | (b >> 1); }

// Activation planes in LDS: element e = 256*sb + E of column `col` sits at
// half index ((((sb*8 + t)*4 + g)*NC + col) << 3) + pos with
//   piece = 2*(E >> 6) + ((E >> 4) & 1)   (16-byte piece of the code bytes that holds its nibble)
//   g = piece & 3, slot = piece >> 2       (lane group that loads the piece; first or second load)
//   t = slot*4 + ((E >> 5) & 1)*2 + ((E >> 3) & 1)   (which of the lane's eight MFMAs)
//   pos = 4*((E >> 2) & 1) + kslot_of_byte(E & 3)
// so that lane (col, g) reads its 8 k-slots of MFMA t with one 128-bit load.

// index (in halfs) of the sum of sub-block j of superblock sb
__device__ __forceinline__ uint32_t s_slot(uint32_t sb, uint32_t j, uint32_t nc, uint32_t col) {
    return ((((sb * 2u + (j >> 2)) * nc) + col) << 2) + kslot_of_byte(j & 3u);
}

struct q4k_regs {
    lev_u4 hdr, a, b;
};

__device__ __forceinline__ void q4k_issue(const uint8_t *__restrict__ w, uint64_t row_bytes, uint32_t row,
                                          uint32_t sb, uint32_t g, q4k_regs &r) {
    const uint8_t *p = w + (uint64_t)row * row_bytes + (uint64_t)sb * 144u;
    r.hdr = *reinterpret_cast<const lev_u4 *>(p);
    r.a = *reinterpret_cast<const lev_u4 *>(p + 16u + 16u * g);
    r.b = *reinterpret_cast<const lev_u4 *>(p + 80u + 16u * g);
}

// Four MFMA pairs for one 16-byte piece: scale `sc_lo` for its low nibbles
// (sub-block 2c), `sc_hi` for its high nibbles (sub-block 2c+1).
template <int NC>
__device__ __forceinline__ lev_f32x4 q4k_piece(lev_u4 P, uint32_t sc_lo, uint32_t sc_hi,
                                               const _Float16 *__restrict__ xh,
                                               const _Float16 *__restrict__ xl, uint32_t base,
                                               lev_f32x4 acc) {
    // base: half index of (sb, t = slot*4, g, col); t advances by 4*NC*8 halfs
    constexpr uint32_t kStrideT = 4u * NC * 8u;
#pragma unroll
    for (int nib = 0; nib < 2; ++nib) {
        const uint32_t sc = nib ? sc_hi : sc_lo;
#pragma unroll
        for (int dp = 0; dp < 2; ++dp) {
            uint32_t d0 = P[2 * dp], d1 = P[2 * dp + 1];
            if (nib) {
                d0 >>= 4;
                d1 >>= 4;
            }
            lev_u4 bits;
            bits.x = __umul24(d0 & 0x000F000Fu, sc);
            bits.y = __umul24((d0 >> 8) & 0x000F000Fu, sc);
            bits.z = __umul24(d1 & 0x000F000Fu, sc);
            bits.w = __umul24((d1 >> 8) & 0x000F000Fu, sc);
            const lev_h8 B = __builtin_bit_cast(lev_h8, bits);
            const uint32_t at = base + (uint32_t)(nib * 2 + dp) * kStrideT;
            const lev_h8 Ah = *reinterpret_cast<const lev_h8 *>(xh + at);
            const lev_h8 Al = *reinterpret_cast<const lev_h8 *>(xl + at);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(Ah, B, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(Al, B, acc, 0, 0, 0);
        }
    }
    return acc;
}

// NC: columns the LDS layout holds (1, 2, 4 or 8; >= ncol).
// SHORT: no wave has more than three tasks (every decode-sized matrix); the
// kernel is then straight-line code, so the wait before each task covers
// exactly that task's loads and the first task is multiplied while the other
// two are still streaming in.  In the general kernel's loop the compiler's wait
// counts, merged over the back edge, make a task wait for most of what is in
// flight, which costs little once a wave has many tasks.
template <int NC, bool SHORT>
__global__ void __launch_bounds__(kMThreads)
q4_k_mfma_gemv(const uint8_t *__restrict__ w, const float *__restrict__ x,
               const float *__restrict__ gain, float eps, float *__restrict__ y, uint32_t cols,
               uint32_t rows, uint32_t ncol) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const uint32_t SB = cols >> 8;
    const uint32_t plane = SB * NC * 256u;                 // halfs per activation plane
    _Float16 *xh = reinterpret_cast<_Float16 *>(smem);
    _Float16 *xl = xh + plane;
    _Float16 *sh = xl + plane;                             // sub-block sums, high / low
    _Float16 *sl = sh + SB * NC * 8u;
    float *part = reinterpret_cast<float *>(sl + SB * NC * 8u);   // [2][wave][row][NC]
    float *s_fac = part + 2 * kMWaves * 16 * NC;           // [NC] output factor, [NC] input scale

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;

    // ---- geometry of the weight stream.  The wave's first three tasks are
    // issued once every wave of the workgroup has its activations (a CU's
    // memory pipeline is one queue: weight loads of early waves would hold up
    // the activation loads of late ones); the weights then stream in while the
    // activations are reduced and converted ----
    const uint32_t r = lane & 15u, g = lane >> 4;
    const uint64_t row_bytes = (uint64_t)SB * 144u;
    const uint32_t ngroups = (rows + 15u) >> 4;
    const uint32_t tpr = (SB + kMWaves - 1u) / kMWaves;    // tasks per row group and wave
    const uint32_t ntasks = ((ngroups - blockIdx.x + gridDim.x - 1u) / gridDim.x) * tpr;
    // Branch-free: a task past the end (or past the wave's last superblock)
    // reads the first bytes of the matrix, which stay in cache.
    // A cursor walks the wave's tasks in order: row group rg (stride gridDim.x),
    // within it superblock wave + 16*t for t < tpr.  No divisions.
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

    // ---- stage the activations: x * gain, column scale, fp16 high + low ----
    // A thread takes runs of 8 consecutive elements (the 8 k-slots one lane
    // feeds to one MFMA): two 128-bit loads in, two 128-bit LDS stores out.
    // Slot q = tid + i*1024 is run 4*(q / (4*NC)) + q % 4 of column (q / 4) % NC:
    // four adjacent lanes hold the four runs of one sub-block, and nothing is
    // divided.  A thread's loads are unconditional (clamped) so that they are
    // in flight together; whole passes beyond the data are skipped.
    constexpr int CH = 4;                                   // slots per thread: NC*cols/8 <= 4096
    constexpr uint32_t kLogNC = NC == 8 ? 3u : NC == 4 ? 2u : NC == 2 ? 1u : 0u;
    const uint32_t runs = cols >> 3, subs = cols >> 5, total_slots = runs * NC;
    auto slot_of = [&](uint32_t q, uint32_t &c, uint32_t &k8) {
        c = (q >> 2) & (NC - 1u);
        k8 = ((q >> (2u + kLogNC)) << 2) | (q & 3u);
        return q < total_slots && c < ncol;
    };
    float *s_run = reinterpret_cast<float *>(smem);         // [col][sub-block][2] sum of squares, max: aliases xh
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
#pragma unroll
        for (int i = 0; i < CH; ++i) {
            if ((uint32_t)i * kMThreads >= total_slots) break;
            uint32_t c, k8;
            const bool real = slot_of(tid + (uint32_t)i * kMThreads, c, k8);
            const lev_f32x4 a = va[i], b = vb[i];
            float ss = a.x * a.x;
            ss = fmaf(a.y, a.y, ss); ss = fmaf(a.z, a.z, ss); ss = fmaf(a.w, a.w, ss);
            ss = fmaf(b.x, b.x, ss); ss = fmaf(b.y, b.y, ss); ss = fmaf(b.z, b.z, ss); ss = fmaf(b.w, b.w, ss);
            if (gain) {
                va[i] = a * ga[i];
                vb[i] = b * gb[i];
            }
            const lev_f32x4 p = va[i], r2 = vb[i];
            float mx = fmaxf(fmaxf(fabsf(p.x), fabsf(p.y)), fmaxf(fabsf(p.z), fabsf(p.w)));
            mx = fmaxf(mx, fmaxf(fmaxf(fabsf(r2.x), fabsf(r2.y)), fmaxf(fabsf(r2.z), fabsf(r2.w))));
            // the four runs of a sub-block sit in four adjacent lanes
            ss = lev_group_sum<4>(ss);
            mx = fmaxf(mx, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
                               0, __builtin_bit_cast(int, mx), 0xB1, 0xF, 0xF, true)));
            mx = fmaxf(mx, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
                               0, __builtin_bit_cast(int, mx), 0x4E, 0xF, 0xF, true)));
            if (real && (k8 & 3u) == 3u) {
                s_run[2u * (c * subs + (k8 >> 2))] = ss;
                s_run[2u * (c * subs + (k8 >> 2)) + 1u] = mx;
            }
        }
    }
    lev_barrier_lds();
    issue(ci, W0);
    issue(ci, W1);
    issue(ci, W2);
    // one wave per column adds the column's sub-block sums in a fixed order
    if (wave < ncol) {
        float ss = 0.f, mx = 0.f;
        for (uint32_t k = lane; k < subs; k += 64u) {
            ss += s_run[2u * (wave * subs + k)];
            mx = fmaxf(mx, s_run[2u * (wave * subs + k) + 1u]);
        }
        ss = lev_group_sum<64>(ss);
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
        if (lane == 63u) {
            float inv = 1.0f;
            if (gain) inv = 1.0f / sqrtf(ss / (float)cols + eps);
            // power-of-two scale that brings the column maximum into [1, 2)
            uint32_t ex = (__float_as_uint(mx) >> 23) & 0xFFu;
            if (ex == 0u || ex >= 254u) ex = 127u;          // zero / denormal / non-finite column: no scaling
            s_fac[wave] = inv * __uint_as_float(ex << 23);             // inv_rms * 2^(ex-127)
            s_fac[NC + wave] = __uint_as_float((254u - ex) << 23);     // 2^(127-ex)
        }
    }
    lev_barrier_lds();   // s_run (aliasing xh) is dead from here
#pragma unroll
    for (int i = 0; i < CH; ++i) {
        if ((uint32_t)i * kMThreads >= total_slots) break;
        uint32_t c, k8;
        const bool real = slot_of(tid + (uint32_t)i * kMThreads, c, k8);
        const float scale = s_fac[NC + (real ? c : 0u)];
        const lev_f32x4 a = va[i] * scale, b = vb[i] * scale;
        // k-slot order of the 8 elements: code bytes 0, 2, 1, 3 of each dword
        const float m[8] = {a.x, a.z, a.y, a.w, b.x, b.z, b.y, b.w};
        // packed f32 -> f16 conversions (round to nearest even), residual by a
        // mixed-precision fma: four instructions per two elements
        typedef float f32x2 __attribute__((ext_vector_type(2)));
        typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
        lev_h8 hi, lo;
        float s = 0.f;
#pragma unroll
        for (int k = 0; k < 8; k += 2) {
            const f32x2 pair = {m[k], m[k + 1]};
            const f16x2 h = __builtin_convertvector(pair, f16x2);
            const f32x2 rest = {fmaf((float)h.x, -1.0f, pair.x), fmaf((float)h.y, -1.0f, pair.y)};
            const f16x2 l = __builtin_convertvector(rest, f16x2);
            hi[k] = h.x;
            hi[k + 1] = h.y;
            lo[k] = l.x;
            lo[k + 1] = l.y;
            s += pair.x + pair.y;
        }
        // 4 consecutive runs are one sub-block: its sum for the dmin*m term
        s = lev_group_sum<4>(s);
        if (real) {
            const uint32_t e0 = k8 << 3;
            const uint32_t sb = e0 >> 8, E = e0 & 255u;
            const uint32_t piece = 2u * (E >> 6) + ((E >> 4) & 1u);
            const uint32_t t = (piece >> 2) * 4u + ((E >> 5) & 1u) * 2u + ((E >> 3) & 1u);
            const uint32_t at = (((sb * 8u + t) * 4u + (piece & 3u)) * NC + c) << 3;
            *reinterpret_cast<lev_h8 *>(xh + at) = hi;
            *reinterpret_cast<lev_h8 *>(xl + at) = lo;
            if ((k8 & 3u) == 3u) {
                const uint32_t st = s_slot(sb, (e0 >> 5) & 7u, NC, c);
                const _Float16 shi = (_Float16)s;
                sh[st] = shi;
                sl[st] = (_Float16)(s - (float)shi);
            }
        }
    }
    // columns of the layout beyond ncol hold no data: the A rows that read them
    // (clamped to the last column) only feed outputs that are never stored
    lev_barrier_lds();

    // ---- stream the weights ----
    const uint32_t colc = r < (uint32_t)NC ? r : (uint32_t)NC - 1u;   // A rows past NC: any valid address
    const uint32_t sh16 = 16u * (g >> 1);
    lev_f32x4 yacc = {0.f, 0.f, 0.f, 0.f};

    // One task: superblock task_sb(k) of the 16 rows of group task_rg(k).  After
    // the last task of a row group the waves' partial sums meet in LDS.
    uint32_t parity = 0;
    auto compute = [&](cursor &c, const q4k_regs &W) {
        const uint32_t rg = c.rg, t = c.t;
        const uint32_t sbw = wave + kMWaves * t;
        const bool live = sbw < SB;
        const uint32_t sb = live ? sbw : SB - 1u;

        const uint32_t S0 = W.hdr.y, S1 = W.hdr.z, S2 = W.hdr.w;
        const uint32_t vv = S0 >> sh16, uu = S2 >> sh16;
        const uint32_t scA0 = vv & 63u, scA1 = (vv >> 8) & 63u;
        const uint32_t scB0 = (uu & 0xFu) | ((vv >> 2) & 0x30u);
        const uint32_t scB1 = ((uu >> 8) & 0xFu) | ((vv >> 10) & 0x30u);
        const uint32_t base = (((sb * 8u) * 4u + g) * NC + colc) << 3;
        // two independent accumulator chains, one per piece
        lev_f32x4 acc = {0.f, 0.f, 0.f, 0.f}, accb = {0.f, 0.f, 0.f, 0.f};
        acc = q4k_piece<NC>(W.a, scA0, scA1, xh, xl, base, acc);
        accb = q4k_piece<NC>(W.b, scB0, scB1, xh, xl, base + 4u * (4u * NC * 8u), accb);
        acc += accb;

        // mins: k-slots 0..7 of a 16x16x16 MFMA, lanes g = 0, 1 carry m_0..3, m_4..7
        uint32_t mb = (g & 1u) ? (((S2 >> 4) & 0x0F0F0F0Fu) | ((S1 >> 2) & 0x30303030u))
                               : (S1 & 0x3F3F3F3Fu);
        mb = g >= 2u ? 0u : mb;
        lev_u2 mbits;
        mbits.x = mb & 0x00FF00FFu;
        mbits.y = (mb >> 8) & 0x00FF00FFu;
        const lev_h4 B2 = __builtin_bit_cast(lev_h4, mbits);
        const uint32_t sat = (((sb * 2u + (g & 1u)) * NC) + colc) << 2;
        const lev_h4 A2h = *reinterpret_cast<const lev_h4 *>(sh + sat);
        const lev_h4 A2l = *reinterpret_cast<const lev_h4 *>(sl + sat);
        lev_f32x4 acc2 = {0.f, 0.f, 0.f, 0.f};
        acc2 = __builtin_amdgcn_mfma_f32_16x16x16f16(A2h, B2, acc2, 0, 0, 0);
        acc2 = __builtin_amdgcn_mfma_f32_16x16x16f16(A2l, B2, acc2, 0, 0, 0);

        // both products carry 2^-24 (subnormal bit patterns): fold it into d, dmin;
        // a task past the wave's last superblock contributes nothing
        const float keep = live ? 16777216.0f : 0.0f;
        const float d = lev_f16_bits_to_f32(W.hdr.x & 0xFFFFu) * keep;
        const float dmin = lev_f16_bits_to_f32(W.hdr.x >> 16) * keep;
#pragma unroll
        for (int i = 0; i < 4; ++i) yacc[i] = fmaf(d, acc[i], fmaf(-dmin, acc2[i], yacc[i]));

        if (t + 1u == tpr) {   // workgroup-uniform
            float *pp = part + parity * (kMWaves * 16 * NC);   // two buffers: one barrier per group
            parity ^= 1u;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (4u * g + (uint32_t)i < (uint32_t)NC) pp[(wave * 16u + r) * NC + 4u * g + i] = yacc[i];
            yacc = lev_f32x4{0.f, 0.f, 0.f, 0.f};
            lev_barrier_lds();
            if (tid < 16u * NC) {
                const uint32_t col = tid >> 4, rr = tid & 15u, row = rg * 16u + rr;
                float sum = 0.f;
#pragma unroll
                for (int kk = 0; kk < kMWaves; ++kk) sum += pp[((uint32_t)kk * 16u + rr) * NC + col];
                if (col < ncol && row < rows) y[(uint64_t)col * rows + row] = sum * s_fac[col];
            }
        }
        advance(c);
    };

    // three tasks in flight per wave
    if constexpr (SHORT) {
        compute(cc, W0);
        if (ntasks > 1u) compute(cc, W1);
        if (ntasks > 2u) compute(cc, W2);
        return;
    }
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

size_t q4k_mfma_lds_bytes(uint32_t cols, uint32_t nc) {
    const size_t SB = cols >> 8;
    return 2 * SB * nc * 256 * 2 + 2 * SB * nc * 8 * 2 + (size_t)2 * kMWaves * 16 * nc * 4 +
           (size_t)2 * nc * 4;
}

template <int NC, bool SHORT>
hipError_t launch_mfma_variant(lev_ctx *ctx, const uint8_t *w, const float *x, const float *gain, float eps,
                       float *y, uint32_t cols, uint32_t rows, uint32_t ncol) {
    const size_t lds = q4k_mfma_lds_bytes(cols, NC);
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
                       x, gain, eps, y, cols, rows, ncol);
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

}  // namespace

// Columns one launch of the MFMA kernel can take for this in_dim (0: not usable).
uint32_t lev_q4_k_mfma_cols(const lev_ctx *ctx, uint32_t in_dim) {
    if (in_dim % 256u != 0u || in_dim == 0u) return 0;
    uint32_t nc = 8;
    size_t limit = ctx->props.sharedMemPerBlockOptin > ctx->props.sharedMemPerBlock
                       ? ctx->props.sharedMemPerBlockOptin
                       : ctx->props.sharedMemPerBlock;
    while (nc >= 1u && ((uint64_t)nc * in_dim > 32768u || q4k_mfma_lds_bytes(in_dim, nc) > limit))
        nc >>= 1;
    return nc;
}

// ncol <= lev_q4_k_mfma_cols(ctx, in_dim); w 16-byte aligned.
hipError_t lev_q4_k_mfma_gemv_launch(lev_ctx *ctx, const uint8_t *w, const float *x, const float *gain,
                                     float eps, float *y, uint32_t in_dim, uint32_t rows,
                                     uint32_t ncol) {
    if (ncol > 4) return launch_mfma<8>(ctx, w, x, gain, eps, y, in_dim, rows, ncol);
    if (ncol > 2) return launch_mfma<4>(ctx, w, x, gain, eps, y, in_dim, rows, ncol);
    if (ncol > 1) return launch_mfma<2>(ctx, w, x, gain, eps, y, in_dim, rows, ncol);
    return launch_mfma<1>(ctx, w, x, gain, eps, y, in_dim, rows, ncol);
}

// (RMSNorm +) Q6_K GEMV for one to eight columns of f32 activations on the
// integer matrix cores of gfx950, every sum formed without rounding.
//
// Stands in for g4_q6_matvec / q6k.matvec (Gemma4.swift:4065;
// lev-forge/src/q6k.rs:61-187) applied to nb columns at once as Builder::matvec
// does for Q4_K (rust/crates/lev-model/src/gpu.rs:334-370), with the RMSNorm of
// Builder::norm_quant (gpu.rs:295; rmsnorm, lev-model/src/lib.rs:110-114)
// optionally fused in front, and for the argmax step behind a single column
// (lev-forge/src/ops.rs:479-516).
//
// A Q6_K superblock (Q6.swift:4-62; dequantize_row_q6_K order) is 16 groups of 16
// weights w = d * sc_group * (q - 32), q = ql nibble | qh bit pair << 4.  Element
// 128*half + 32*j + l (j = 0..3, l = 0..31) has its nibble in ql[64*half + 32*(j&1) + l]
// (low for j < 2, high otherwise), its bit pair j in qh[32*half + l], and the scale
// sc[8*half + 2*j + l/16].
//
// Arithmetic, per superblock of a row and column of x:
//   * the activations become integers X = rint(x * 2^(30-e)), 2^e the power of two
//     above the superblock's largest magnitude (|X| <= 2^30: every value within 2^-6
//     of that maximum is represented exactly), written in four balanced base-256
//     digits, the bytes of (X + 0x808080) ^ 0x808080 read as int8: four digit planes;
//   * v_mfma_i32_16x16x64_i8: B = 16 weight rows x 64 codes, each lane group (16
//     lanes) supplying ONE 16-element scale group as bytes 4*(q - 32); A row
//     4*gs + p holds digit plane p of the elements lane group gs supplies and zeros
//     elsewhere, so output row 4*gs + p is the exact sum of 4*(q-32)*digit_p over
//     that one group — and lands in the lane group that loaded the group's codes;
//   * the lane multiplies its four plane sums by the group's int8 scale and adds
//     them up over the superblock in 32-bit integers (|sum| < 2^29), then recombines
//     the planes in f64 (below 2^53: exact) and applies d and the power of two;
//   * partial sums of a row (lane groups, waves) are added in f64 and rounded to
//     f32 once.
// Nothing depends on the order of the additions.
//
// lane (r, g) = (l % 16, l / 16) multiplies weight row r of the task's 16 rows, chunk g
// of the superblock = ql bytes [32g, 32g+32) (half g/2, j in {g%2, g%2 + 2}) with the 32
// qh bytes of that half, 8 scale bytes and d.  The bytes do not come from memory in that
// shape: the L1 takes one tag lookup per 64 bytes a group of four lanes touches, and
// with one row per lane (16 bytes here, 16 bytes 3360 bytes further on) every lane is a
// lookup of its own (measured: 27 M lookups per launch, one per CU and clock, 39 us).
// So a load instruction reads 4 rows x 256 contiguous bytes (16 lanes x 16 bytes per
// row: the superblock's 210 bytes), four of them a task, and the wave turns the
// pieces round through a private LDS area (written as loaded, read per (row, chunk);
// pieces rotated by 4 per row and a 16-byte skew per instruction keep both sides
// free of bank conflicts).
//
// Workgroup = 16 waves.  Several columns (q6_k_mfma_gemv): S waves share a group of 16
// rows (each takes 1/S of the row's superblocks), 16/S row groups per workgroup and
// round; the digit planes of every column are staged once per workgroup; the partial
// sums of a round meet in LDS.  One column of at most sixteen superblocks
// (q6_k_mfma_gemv_one): a wave per superblock column, see there.  A NaN or infinity in a column of x makes every output of
// that column NaN.
#include "lev_common.hpp"
#include "top2.hpp"

#include <cstdlib>

namespace {

constexpr int kQThreads = 1024;
constexpr int kQWaves = kQThreads / LEV_WAVE;
constexpr uint32_t kQZeroBytes = 512;   // what masked lanes read as their A operand

typedef int q6m_i4 __attribute__((ext_vector_type(4)));
struct __attribute__((packed, aligned(2))) q6m_u4 { uint32_t v[4]; };
struct __attribute__((packed, aligned(2))) q6m_u2 { uint32_t v[2]; };

constexpr uint32_t kQAreaStride = 1024 + 16;              // one load instruction's pieces + skew
constexpr uint32_t kQAreaBytes = 4 * kQAreaStride;        // per wave

struct q6m_regs {
    q6m_i4 p[4];   // instruction i: row 4i + l/16, piece (l%16 - 4*(l/16)) % 16 of its superblock
};

// Byte offset, from the start of a superblock, of the piece a lane loads.  Superblocks are
// 210 bytes: even ones start on a dword boundary, odd ones two bytes past one, and a 16-byte
// load from such an address costs the L1 several lookups (4 us of 29 at 32000 x 4096).  So
// the 14 pieces of an odd superblock start 14 bytes early, at [-14 + 16p, +16): dword
// aligned, ending exactly at the block's end, the logical piece P = bytes [16P, 16P+16) being
// the last two bytes of piece P and the first 14 of piece P+1.  An even superblock's pieces
// are [16p, +16) for p < 13.  Piece 13 is bytes [194, 210) for both, so that d is its last
// two bytes and nothing behind the block is read (for an even superblock that one piece is
// off the dword boundary).  Lanes 14 and 15 of a row repeat piece 1: never used.
__device__ __forceinline__ int32_t q6m_piece_offset(uint32_t lane, uint32_t odd) {
    const uint32_t p = ((lane & 15u) - 4u * (lane >> 4)) & 15u;
    if (p == 13u) return 194;
    return (int32_t)(16u * (p < 13u ? p : 1u)) - (odd ? 14 : 0);
}

__device__ __forceinline__ void q6m_issue(const uint8_t *__restrict__ w, uint64_t row_bytes, uint32_t row0,
                                          uint32_t rows, uint32_t sb, uint32_t lane, int32_t poff,
                                          q6m_regs &R) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        uint32_t row = row0 + 4u * (uint32_t)i + (lane >> 4);
        row = row < rows ? row : rows - 1u;
        const q6m_u4 v = *reinterpret_cast<const q6m_u4 *>(
            w + (uint64_t)row * row_bytes + (uint64_t)(int64_t)((int32_t)(sb * 210u) + poff));
        R.p[i] = q6m_i4{(int)v.v[0], (int)v.v[1], (int)v.v[2], (int)v.v[3]};
    }
}

// What a lane needs to turn a task's pieces into its matrix-core operands.
// lane (r, g): weight row r of the task's 16, chunk g of the superblock (half hf = g/2,
// j in {jb, jb + 2} with jb = g%2).  `odd`: the wave's superblocks are the odd ones.
struct q6m_lane {
    uint8_t *area;                // the wave's turn-round area
    uint32_t lane, sel, maskq;
    uint32_t rot[2];              // rotate right: bit pair jb + 2*nb of a qh byte to bits 6..7
    uint32_t scoff[2];            // bit offset of scale 2*jb + lh in its dword
    uint32_t at_ql[2], c3_ql[2], at_qh[2], c3_qh[2], at_sc[3], at_d;

    // area_all + wave * stride: the wave's turn-round area (kQAreaBytes of it)
    __device__ __forceinline__ q6m_lane(uint8_t *area_all, uint32_t wave, uint32_t lane_, uint32_t odd,
                                        uint32_t stride = kQAreaBytes)
        : area(area_all + wave * stride), lane(lane_) {
        const uint32_t r = lane & 15u, g = lane >> 4, hf = g >> 1, jb = g & 1u;
        maskq = jb ? 0xCCCCCCCCu : 0x33333333u;   // the bit pairs jb and jb+2 of a qh byte
        rot[0] = 26u + 2u * jb;
        rot[1] = (30u + 2u * jb) & 31u;
        scoff[0] = 16u * jb;
        scoff[1] = 16u * jb + 8u;
        // where (row r, piece P) of a task sits in the area: instruction r/4 wrote row r%4's
        // pieces to lanes 16*(r%4) + (P + 4*(r%4)) % 16
        auto piece_at = [&](uint32_t P) {
            return (r >> 2) * kQAreaStride + (16u * (r & 3u) + ((P + 4u * (r & 3u)) & 15u)) * 16u;
        };
        // logical piece P: an even wave reads piece P; an odd one piece P+1 and, for its first
        // two bytes, the last dword of piece P.  `sel` picks per byte from {next, previous} dword.
        sel = odd ? 0x05040302u : 0x07060504u;
        at_ql[0] = piece_at(2u * g + odd);
        at_ql[1] = piece_at(2u * g + 1u + odd);
        at_qh[0] = piece_at(8u + 2u * hf + odd);
        at_qh[1] = piece_at(9u + 2u * hf + odd);
        c3_ql[0] = piece_at(2u * g) + 12u;
        c3_ql[1] = piece_at(2u * g + 1u) + 12u;
        c3_qh[0] = piece_at(8u + 2u * hf) + 12u;
        c3_qh[1] = piece_at(9u + 2u * hf) + 12u;
        // the eight scale bytes 192 + 8*hf ..: three dwords A0..A2, the wanted two being
        // {A1, A2} (even) or the bytes 2.. of {A0, A1, A2} (odd: stream position 206 + 8*hf)
        at_sc[0] = odd ? (hf ? piece_at(13u) + 4u : piece_at(12u) + 12u) : piece_at(12u);
        at_sc[1] = odd ? (hf ? piece_at(13u) + 8u : piece_at(13u)) : piece_at(12u) + 8u * hf;
        at_sc[2] = odd ? (hf ? piece_at(13u) + 12u : piece_at(13u) + 4u) : piece_at(12u) + 8u * hf + 4u;
        at_d = piece_at(13u) + 14u;
    }

    // B operands of the four MFMAs of a task (nb = nibble, lh = which 16 of the chunk's 32
    // bytes): byte = nibble << 2 | bit pair << 6 with bit 7 flipped = 4*(q - 32) as int8.  The
    // qh dwords are cleaned once (both pairs this lane uses survive, their top bits flipped);
    // rotated so that the wanted pair sits in bits 6..7 the other one falls into bits 2..3,
    // which the merge takes from the nibbles.  sc[nb][lh]: the int8 scale of the 16 weights.
    __device__ __forceinline__ void operands(const q6m_regs &W, q6m_i4 (&B)[2][2], int (&sc)[2][2],
                                             uint32_t &dbits) const {
        // the task's pieces go round through the wave's area: written as loaded, read as
        // (row r, chunk g) wants them.  One wave's LDS operations run in order.
#pragma unroll
        for (int i = 0; i < 4; ++i)
            *reinterpret_cast<q6m_i4 *>(area + (uint32_t)i * kQAreaStride + lane * 16u) = W.p[i];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        auto piece = [&](uint32_t at, uint32_t c3) {
            const q6m_i4 n = *reinterpret_cast<const q6m_i4 *>(area + at);
            const uint32_t prev = *reinterpret_cast<const uint32_t *>(area + c3);
            return q6m_i4{(int)__builtin_amdgcn_perm((uint32_t)n.x, prev, sel),
                          (int)__builtin_amdgcn_perm((uint32_t)n.y, (uint32_t)n.x, sel),
                          (int)__builtin_amdgcn_perm((uint32_t)n.z, (uint32_t)n.y, sel),
                          (int)__builtin_amdgcn_perm((uint32_t)n.w, (uint32_t)n.z, sel)};
        };
        const q6m_i4 ql[2] = {piece(at_ql[0], c3_ql[0]), piece(at_ql[1], c3_ql[1])};
        const q6m_i4 qh[2] = {piece(at_qh[0], c3_qh[0]), piece(at_qh[1], c3_qh[1])};
        const uint32_t sa0 = *reinterpret_cast<const uint32_t *>(area + at_sc[0]);
        const uint32_t sa1 = *reinterpret_cast<const uint32_t *>(area + at_sc[1]);
        const uint32_t sa2 = *reinterpret_cast<const uint32_t *>(area + at_sc[2]);
        const uint32_t scw[2] = {__builtin_amdgcn_perm(sa1, sa0, sel), __builtin_amdgcn_perm(sa2, sa1, sel)};
        dbits = *reinterpret_cast<const uint16_t *>(area + at_d);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();   // the reads are issued before the next task's writes
#pragma unroll
        for (int lh = 0; lh < 2; ++lh) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint32_t qc = ((uint32_t)qh[lh][i] ^ 0xAAAAAAAAu) & maskq;
#pragma unroll
                for (int nb = 0; nb < 2; ++nb) {
                    const uint32_t nib = nb ? (uint32_t)ql[lh][i] >> 2 : (uint32_t)ql[lh][i] << 2;
                    const uint32_t top = __builtin_amdgcn_alignbit(qc, qc, rot[nb]);
                    B[nb][lh][i] = (int)((nib & 0x3C3C3C3Cu) | (top & ~0x3C3C3C3Cu));
                }
            }
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) sc[nb][lh] = __builtin_amdgcn_sbfe((int)scw[nb], scoff[lh], 8u);
        }
    }
};

// LDS, for SB superblocks and NC columns:
//   dig  [NC][16*SB groups][4 planes][16 bytes]
//   zero [512 bytes]
//   psb  [NC][SB] f64     2^(e-32) per superblock (the 4 of the codes included)
//   ssq  [NC][SB] f64     sums of squares (RMSNorm)
//   part [pb][16 waves][16 rows][NC] f64
//   inv  [NC] f64, bad [NC] u32
//   area [16 waves][4 x (1024 + 16) bytes]           the weights of a task on their way round
template <int NC>
struct q6m_lds {
    static __host__ __device__ size_t dig_bytes(uint32_t cols) { return (size_t)NC * cols * 4u; }
    static __host__ __device__ size_t total(uint32_t cols, uint32_t pb) {
        return dig_bytes(cols) + kQZeroBytes + (size_t)2 * NC * (cols >> 8) * 8u +
               (size_t)pb * kQWaves * 16u * NC * 8u + (size_t)NC * 16u + (size_t)kQWaves * kQAreaBytes;
    }
};

// The greedy token behind one column: `best` is the running top two of the rows this thread
// stored (waves 0 .. nred-1 hold candidates).  Every thread of the workgroup calls it.
__device__ __forceinline__ void q6m_greedy_token(top2 best, uint32_t nred, lev_f32x4 *__restrict__ partials,
                                                 uint32_t *__restrict__ tickets, uint32_t *__restrict__ out_idx,
                                                 float *__restrict__ out_margin) {
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    __shared__ float s_best[kQWaves], s_second[kQWaves];
    __shared__ uint32_t s_idx[kQWaves];
    // only the waves that stored outputs hold candidates; wave 0 finishes alone, so that no
    // wave waits at a barrier for another one's stores
    if (wave < nred) {
        best = top2_wave(best);
        if (lane == 0u) {
            s_best[wave] = best.best;
            s_second[wave] = best.second;
            s_idx[wave] = best.idx;
        }
    }
    lev_barrier_lds();
    if (wave != 0u) return;
    top2 m{s_best[0], s_second[0], s_idx[0]};
    if (nred > 1u) {   // workgroup-uniform
        m = top2{kTop2Floor, kTop2Floor, 0xFFFFFFFFu};
        if (lane < nred) m = top2{s_best[lane], s_second[lane], s_idx[lane]};
        m = top2_wave(m);
    }
    if (!tickets) {
        if (lane == 0u)
            partials[blockIdx.x] = lev_f32x4{m.best, m.second, __builtin_bit_cast(float, m.idx), 0.f};
        return;
    }
    // The last workgroup to finish merges the partials (a kernel of its own for that costs a
    // launch and a cold round trip: 7 us behind a 25 us GEMV).  The partial goes out in
    // device-scope stores, which go through to memory, and the arrival is counted once they
    // have completed (a fence here would write back every dirty line of the L2, the rows of y
    // included: 250 of those cost 12 us).  Arrivals are counted in four groups (workgroup
    // index mod 4, counters 4 KB apart: arrivals at one word are served one after the other, some
    // ten nanoseconds each, and the workgroups of a resident grid finish within a microsecond of
    // each other); the last of each group arrives at a fifth counter.  (Eight groups: 0.4 us
    // slower at 250 workgroups, the second level then waits for more stragglers; one: the same
    // as four there, and a queue of 250 in the worst case.)
    uint32_t last = 0u;
    if (lane == 0u) {
        float *pf = reinterpret_cast<float *>(partials + blockIdx.x);
        __hip_atomic_store(pf, m.best, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(pf + 1, m.second, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(pf + 2, __builtin_bit_cast(float, m.idx), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        lev_publish_wait();
        constexpr uint32_t G = 4u;
        const uint32_t grp = blockIdx.x % G, ngrp = gridDim.x < G ? gridDim.x : G;
        const uint32_t in_grp = (gridDim.x - grp + G - 1u) / G;
        if (__hip_atomic_fetch_add(&tickets[(1u + grp) * 1024u], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) ==
            in_grp - 1u) {
            // nobody else touches the counter before the next launch
            __hip_atomic_store(&tickets[(1u + grp) * 1024u], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (__hip_atomic_fetch_add(&tickets[0], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == ngrp - 1u) {
                __hip_atomic_store(&tickets[0], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                last = 1u;
            }
        }
    }
    if (!__builtin_amdgcn_readfirstlane((int)last)) return;
    top2 f{kTop2Floor, kTop2Floor, 0xFFFFFFFFu};
    const float *pf = reinterpret_cast<const float *>(partials);
    // device-scope loads: the other workgroups' partials come from beyond this XCD's L2.  Four
    // records a lane are requested together (256 workgroups: one trip to memory, not four)
    for (uint32_t i0 = lane; i0 < gridDim.x; i0 += 256u) {
        float b[4], s2[4], ib[4];
#pragma unroll
        for (uint32_t u = 0; u < 4u; ++u) {
            const uint32_t i = i0 + 64u * u < gridDim.x ? i0 + 64u * u : i0;
            b[u] = __hip_atomic_load(pf + 4u * i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            s2[u] = __hip_atomic_load(pf + 4u * i + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            ib[u] = __hip_atomic_load(pf + 4u * i + 2u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
#pragma unroll
        for (uint32_t u = 0; u < 4u; ++u)   // (a request past the end repeated the lane's first record: not merged again)
            if (i0 + 64u * u < gridDim.x) f = top2_merge(f, top2{b[u], s2[u], __float_as_uint(ib[u])});
    }
    f = top2_wave(f);
    if (lane == 0u) {
        if (out_idx) out_idx[0] = f.idx == 0xFFFFFFFFu ? 0u : f.idx;   // nothing above -inf: first
        if (out_margin) out_margin[0] = f.best - f.second;
    }
}

// NC: columns staged (1, 2, 4 or 8; >= ncol).  S: waves per row group (2..16, a
// power of two).  partials (optional, ncol == 1): the workgroup's top two outputs.
template <int NC>
__global__ void __launch_bounds__(kQThreads)
q6_k_mfma_gemv(const uint8_t *__restrict__ w, const float *__restrict__ x, const float *__restrict__ gain,
               float eps, float *__restrict__ y, uint32_t cols, uint32_t rows, uint32_t ncol, uint32_t S,
               uint32_t pb, double rcols, lev_f32x4 *__restrict__ partials, uint32_t *__restrict__ tickets,
               uint32_t *__restrict__ out_idx, float *__restrict__ out_margin) {
    using L = q6m_lds<NC>;
    constexpr uint32_t kLogNC = NC == 8 ? 3u : NC == 4 ? 2u : NC == 2 ? 1u : 0u;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const uint32_t SB = cols >> 8;
    uint8_t *dig = smem;
    uint8_t *zero = smem + L::dig_bytes(cols);
    double *psb = reinterpret_cast<double *>(zero + kQZeroBytes);
    double *ssq = psb + (size_t)NC * SB;
    double *part = ssq + (size_t)NC * SB;
    double *s_inv = part + (size_t)pb * kQWaves * 16u * NC;
    uint32_t *s_bad = reinterpret_cast<uint32_t *>(s_inv + NC);
    uint8_t *area_all = reinterpret_cast<uint8_t *>(s_inv) + (size_t)NC * 16u;

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;

    // ---- geometry of the weight stream ----
    const uint32_t r = lane & 15u, g = lane >> 4;
    const uint64_t row_bytes = (uint64_t)SB * 210u;
    const uint32_t ngroups = (rows + 15u) >> 4;
    const uint32_t slots = kQWaves / S;                    // row groups per workgroup and round
    const uint32_t slot = wave / S, kpart = wave % S;
    const uint32_t tpr = (SB + S - 1u) / S;                // tasks per round and wave
    const uint32_t wgrounds = (ngroups + slots - 1u) / slots;
    const uint32_t nrounds = (wgrounds - blockIdx.x + gridDim.x - 1u) / gridDim.x;
    const uint32_t ntasks = nrounds * tpr;
    // A cursor walks the wave's tasks in order: round rd, within it superblock
    // kpart + S*t for t < tpr (S is even: all of a wave's superblocks are even or all odd).
    // A task past the end reads the first bytes of the matrix.
    struct cursor {
        uint32_t k, rd, t;
    };
    auto advance = [&](cursor &c) {
        ++c.k;
        if (++c.t == tpr) {
            c.t = 0;
            ++c.rd;
        }
    };
    const uint32_t odd = kpart & 1u;
    const int32_t poff = q6m_piece_offset(lane, odd), poff_even = q6m_piece_offset(lane, 0u);
    auto group_of = [&](uint32_t rd, uint32_t sl) { return (rd * gridDim.x + blockIdx.x) * slots + sl; };
    auto issue = [&](cursor &c, q6m_regs &W) {
        const uint32_t sbw = kpart + S * c.t;
        const bool real = c.k < ntasks && sbw < SB;
        // (past the end: the first superblock of the matrix, pieces as for an even one)
        q6m_issue(w, row_bytes, real ? group_of(c.rd, slot) * 16u : 0u, rows, real ? sbw : 0u, lane,
                  real ? poff : poff_even, W);
        advance(c);
    };
    cursor ci{0u, 0u, 0u}, cc{0u, 0u, 0u};
    q6m_regs W0, W1, W2;

    // ---- stage the activations ----
    // A wave takes one superblock of one column per pass (unit u = wave + 16*i: column
    // u / SB, superblock u % SB), a lane four consecutive elements of it.  All loads
    // are requested before the first is used; passes beyond the data are skipped.
    constexpr int CH = 8;                                   // passes: NC*cols <= 32768
    const uint32_t units = ncol * SB;
    lev_f32x4 v[CH];
    if (tid < (uint32_t)NC) s_bad[tid] = 0u;
    if (tid < kQZeroBytes / 4u) reinterpret_cast<uint32_t *>(zero)[tid] = 0u;
    {
        lev_f32x4 gv[CH];
#pragma unroll
        for (int i = 0; i < CH; ++i) {
            if ((uint32_t)i * kQWaves >= units) break;      // workgroup-uniform
            const uint32_t u = wave + (uint32_t)i * kQWaves;
            const uint32_t uc = u < units ? u : 0u;
            const uint32_t c = uc / SB, sb = uc % SB;
            v[i] = reinterpret_cast<const lev_f32x4 *>(x + (uint64_t)c * cols)[sb * 64u + lane];
            if (gain) gv[i] = reinterpret_cast<const lev_f32x4 *>(gain)[sb * 64u + lane];
        }
        if (gain) {
            // RMSNorm as the reference computes it: mean square and 1/sqrt in f64, then
            // (f32)(x * inv) * gain
#pragma unroll
            for (int i = 0; i < CH; ++i) {
                if ((uint32_t)i * kQWaves >= units) break;
                const uint32_t u = wave + (uint32_t)i * kQWaves;
                const lev_f32x4 a = v[i];
                double ss = (double)a.x * (double)a.x;
                ss = fma((double)a.y, (double)a.y, ss);
                ss = fma((double)a.z, (double)a.z, ss);
                ss = fma((double)a.w, (double)a.w, ss);
                ss = lev_group_sum_f64<64>(ss);
                if (lane == 63u && u < units) ssq[u] = ss;   // u = c*SB + sb
            }
        }
        // every wave of the workgroup has its activations before the first weights are
        // requested: a CU's memory pipeline is one queue
        lev_barrier_lds();
        issue(ci, W0);
        if (gain) {
            if (wave < ncol) {
                double ss = 0.0;
                for (uint32_t k = lane; k < SB; k += 64u) ss += ssq[wave * SB + k];
                ss = lev_group_sum_f64<64>(ss);
                // 1/sqrt(mean + eps): the hardware estimate and two Newton steps (full f64 accuracy)
                const double a = fma(ss, rcols, (double)eps);
                double rs = __builtin_amdgcn_rsq(a);
                rs = rs * fma(-0.5 * a * rs, rs, 1.5);
                rs = rs * fma(-0.5 * a * rs, rs, 1.5);
                if (lane == 63u) s_inv[wave] = rs;
            }
            lev_barrier_lds();
#pragma unroll
            for (int i = 0; i < CH; ++i) {
                if ((uint32_t)i * kQWaves >= units) break;
                const uint32_t u = wave + (uint32_t)i * kQWaves;
                const double inv = s_inv[u < units ? u / SB : 0u];
#pragma unroll
                for (int k = 0; k < 4; ++k) v[i][k] = (float)((double)v[i][k] * inv) * gv[i][k];
            }
        }
    }
#pragma unroll
    for (int i = 0; i < CH; ++i) {
        if ((uint32_t)i * kQWaves >= units) break;
        const uint32_t u = wave + (uint32_t)i * kQWaves;
        const bool real = u < units;
        const uint32_t c = real ? u / SB : 0u, sb = real ? u % SB : 0u;
        const lev_f32x4 a = v[i];
        const float e4[4] = {a.x, a.y, a.z, a.w};
        // largest magnitude of the superblock as an integer: NaN and infinity sort above every number
        uint32_t mb = 0u;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint32_t bits = __float_as_uint(e4[k]) & 0x7FFFFFFFu;
            mb = bits > mb ? bits : mb;
        }
        mb = lev_row16_max_u32(mb);   // all 16 lanes of a row hold the row's maximum
        {
            const uint32_t m0 = (uint32_t)__builtin_amdgcn_readlane((int)mb, 0);
            const uint32_t m1 = (uint32_t)__builtin_amdgcn_readlane((int)mb, 16);
            const uint32_t m2 = (uint32_t)__builtin_amdgcn_readlane((int)mb, 32);
            const uint32_t m3 = (uint32_t)__builtin_amdgcn_readlane((int)mb, 48);
            const uint32_t ma = m0 > m1 ? m0 : m1, mc = m2 > m3 ? m2 : m3;
            mb = ma > mc ? ma : mc;
        }
        uint32_t ex = mb >> 23;                             // biased exponent: |x| < 2^(ex-126)
        if (real && ex == 255u && lane == 0u) atomicOr(&s_bad[c], 1u);
        ex = ex < 30u ? 30u : (ex > 254u ? 254u : ex);      // keeps both powers of two normal numbers
        const float scale = __uint_as_float((283u - ex) << 23);   // 2^(156-ex): |x*scale| < 2^30
        uint32_t Y[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int X = (int)rintf(e4[k] * scale);
            // balanced base-256 digits: adding 0x80 to each of the low three bytes carries into
            // the next digit where a byte exceeds 127, and flipping bit 7 subtracts it again
            Y[k] = ((uint32_t)X + 0x00808080u) ^ 0x00808080u;
        }
        // 4x4 byte transpose: digit k of the four elements in one dword, element 0 lowest
        const uint32_t t0 = __builtin_amdgcn_perm(Y[1], Y[0], 0x05010400u);   // a0 b0 a1 b1
        const uint32_t t1 = __builtin_amdgcn_perm(Y[1], Y[0], 0x07030602u);   // a2 b2 a3 b3
        const uint32_t t2 = __builtin_amdgcn_perm(Y[3], Y[2], 0x05010400u);
        const uint32_t t3 = __builtin_amdgcn_perm(Y[3], Y[2], 0x07030602u);
        const uint32_t dw[4] = {__builtin_amdgcn_perm(t2, t0, 0x05040100u), __builtin_amdgcn_perm(t2, t0, 0x07060302u),
                                __builtin_amdgcn_perm(t3, t1, 0x05040100u), __builtin_amdgcn_perm(t3, t1, 0x07060302u)};
        if (real) {
            // group 16*sb + lane/4, plane p at +16p, the lane's four elements at +4*(lane%4)
            uint8_t *at = dig + (size_t)c * cols * 4u + (size_t)(16u * sb + (lane >> 2)) * 64u + 4u * (lane & 3u);
#pragma unroll
            for (int p = 0; p < 4; ++p) *reinterpret_cast<uint32_t *>(at + 16 * p) = dw[p];
            if (lane == 0u) psb[c * SB + sb] = __hiloint2double((int)((ex + 865u) << 20), 0);   // 2^(ex-158)
        }
    }
    // columns of the layout beyond ncol hold no data: they only feed outputs that are never stored
    lev_barrier_lds();

    // ---- stream the weights ----
    const uint32_t hf = g >> 1, jb = g & 1u;
    const bool feeds = (r >> 2) == g;                      // this lane's A row belongs to its own lane group
    const q6m_lane L6(area_all, wave, lane, odd);
    double yacc[NC];
#pragma unroll
    for (int q = 0; q < NC; ++q) yacc[q] = 0.0;
    top2 best{kTop2Floor, kTop2Floor, 0xFFFFFFFFu};

    uint32_t parity = 0;
    auto compute = [&](cursor &c, const q6m_regs &W) {
        const uint32_t rd = c.rd, t = c.t;
        const uint32_t sbw = kpart + S * t;
        const bool live = sbw < SB;
        const uint32_t sb = live ? sbw : SB - 1u;
        q6m_i4 B[2][2];
        int sc[2][2];
        uint32_t dbits;
        L6.operands(W, B, sc, dbits);
        // a task past the wave's last superblock contributes nothing
        const double d = live ? (double)lev_f16_bits_to_f32(dbits) : 0.0;
        // lane (r, g) feeds A row r = 4*gs + p: plane p of group 16*sb + 8*hf + 2*jb (+ 4*nb + lh)
        // when gs == g, zeros otherwise
        const uint32_t aoff = (uint32_t)((16u * sb + 8u * hf + 2u * jb) * 64u + 16u * (r & 3u));
#pragma unroll
        for (int q = 0; q < NC; ++q) {
            const uint8_t *ab = feeds ? dig + (size_t)q * cols * 4u + aoff : zero;
            int E[4] = {0, 0, 0, 0};
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) {
#pragma unroll
                for (int lh = 0; lh < 2; ++lh) {
                    const q6m_i4 A = *reinterpret_cast<const q6m_i4 *>(ab + (4 * nb + lh) * 64);
                    const q6m_i4 D =
                        __builtin_amdgcn_mfma_i32_16x16x64_i8(A, B[nb][lh], q6m_i4{0, 0, 0, 0}, 0, 0, 0);
                    // |D| <= 16*128*128 = 2^18, |sc| <= 2^7: four products per plane stay below 2^27
#pragma unroll
                    for (int p = 0; p < 4; ++p) {
                        E[p] += __mul24(D[p], sc[nb][lh]);
                        asm("" : "+v"(E[p]));   // one multiply-add per plane: keeps the sums from being regrouped
                    }
                }
            }
            const double hi = fma((double)E[3], 256.0, (double)E[2]);
            const double lo = fma((double)E[1], 256.0, (double)E[0]);
            const double dot = fma(hi, 65536.0, lo);
            yacc[q] = fma(psb[q * SB + sb] * d, dot, yacc[q]);
        }

        if (t + 1u == tpr) {   // workgroup-uniform: the round ends
            double *pp = part + parity * (kQWaves * 16u * NC);
            parity ^= pb - 1u;
#pragma unroll
            for (int q = 0; q < NC; ++q) {
                double s = yacc[q];
                s += __shfl_xor(s, 16);
                s += __shfl_xor(s, 32);
                if (g == 0u) pp[(wave * 16u + r) * NC + q] = s;
                yacc[q] = 0.0;
            }
            lev_barrier_lds();
            for (uint32_t i = tid; i < slots * 16u * NC; i += kQThreads) {
                const uint32_t rr = i & 15u, col = (i >> 4) & (NC - 1u), sl = i >> (4u + kLogNC);
                const uint32_t row = group_of(rd, sl) * 16u + rr;
                double sum = 0.0;
                for (uint32_t k = 0; k < S; ++k) sum += pp[((sl * S + k) * 16u + rr) * NC + col];
                if (col < ncol && row < rows) {
                    const float out = s_bad[col] ? __builtin_nanf("") : (float)sum;
                    y[(uint64_t)col * rows + row] = out;
                    // running top two of the rows this thread finishes (rows ascend, so a tie
                    // keeps the earlier, lower index)
                    if (out > best.best) {
                        best.second = best.best;
                        best.best = out;
                        best.idx = row;
                    } else if (out > best.second) {
                        best.second = out;
                    }
                }
            }
            if (pb == 1u) lev_barrier_lds();   // the one buffer is written again by the next round
        }
        advance(c);
    };

    // Three tasks in flight per wave.  The scheduling barriers keep a refill's loads
    // behind the compute that frees its registers: hoisted above it they would be
    // younger than the data the compute waits for, and the wait would cover them too.
    issue(ci, W1);
    issue(ci, W2);
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

    if (partials) {
        const uint32_t nred0 = (slots * 16u * NC + 63u) >> 6;
        q6m_greedy_token(best, nred0 < (uint32_t)kQWaves ? nred0 : (uint32_t)kQWaves, partials, tickets, out_idx, out_margin);
    }
}

// ---------------------------------------------------------------------------
// One column, rows of at most sixteen superblocks: a wave per superblock COLUMN of the matrix.
// The wave stages the 256 activations of its column by itself (1 KB of LDS nobody else
// touches), keeps the A operands of its four MFMAs in registers and walks the row groups
// with the next group's weights in flight; the partial sums of a row meet in LDS behind ONE
// barrier per round, nothing but the RMSNorm's sum of squares crosses waves before the
// products.  The arithmetic, the fetch and the turn-round are those of q6_k_mfma_gemv (a
// wave's superblocks are all even or all odd here as well: it has one).
// Two columns go through it as well (a column costs four MFMAs and the recombination again).
// LDS: part [2][16 waves][16 rows][NC] f64 | sums of squares [NC][16] f64 | per wave: turn-round
// area, digit planes [NC][16 groups][4 planes][16 B], a zero strip.
// ---------------------------------------------------------------------------
constexpr uint32_t kQ1DigBytes = 1024u, kQ1ZeroBytes = 16u;
__host__ __device__ constexpr uint32_t q6m_one_part_bytes(uint32_t nc) { return 2u * kQWaves * 16u * 8u * nc; }
__host__ __device__ constexpr uint32_t q6m_one_norm_bytes(uint32_t nc) { return kQWaves * 8u * nc; }
__host__ __device__ constexpr uint32_t q6m_one_wave_bytes(uint32_t nc) { return kQAreaBytes + nc * kQ1DigBytes + kQ1ZeroBytes; }
__host__ __device__ constexpr size_t q6m_one_lds(uint32_t nc) {
    return q6m_one_part_bytes(nc) + q6m_one_norm_bytes(nc) + (size_t)kQWaves * q6m_one_wave_bytes(nc);
}

// wave -> (slot, superblock) as 4-bit entries of two 64-bit kernel arguments (no division in
// front of the first load).  NC: columns staged (1 or 2; >= ncol); one column keeps its A
// operands in registers, several read them from the wave's planes at every product.
// NORM: RMSNorm (gain != nullptr) in front.  partials (optional, ncol == 1): the greedy token.
template <int NC, bool NORM>
__global__ void __launch_bounds__(kQThreads)
q6_k_mfma_gemv_one(const uint8_t *__restrict__ w, const float *__restrict__ x, const float *__restrict__ gain,
                   float eps, float *__restrict__ y, uint32_t cols, uint32_t rows, uint32_t ncol, uint32_t wpr,
                   uint32_t slots, uint64_t slot_of_wave, uint64_t pos_of_wave, double rcols,
                   lev_f32x4 *__restrict__ partials, uint32_t *__restrict__ tickets, uint32_t *__restrict__ out_idx,
                   float *__restrict__ out_margin) {
    constexpr uint32_t kPart = q6m_one_part_bytes(NC), kNorm = q6m_one_norm_bytes(NC), kWave = q6m_one_wave_bytes(NC);
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const uint32_t slot = (uint32_t)(slot_of_wave >> (4u * wave)) & 15u;   // idle waves: slot >= slots
    const uint32_t sb = (uint32_t)(pos_of_wave >> (4u * wave)) & 15u;      // the wave's superblock column
    const uint32_t SB = cols >> 8;

    // the wave's activations first (columns of the layout beyond ncol repeat the last one: never stored) ...
    lev_f32x4 v[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        const uint32_t cc = (uint32_t)c < ncol ? (uint32_t)c : ncol - 1u;
        v[c] = reinterpret_cast<const lev_f32x4 *>(x + (uint64_t)cc * cols)[64u * sb + lane];
    }
    lev_f32x4 gn;
    if (NORM) gn = reinterpret_cast<const lev_f32x4 *>(gain)[64u * sb + lane];
    const bool active = slot < slots;
    const uint64_t row_bytes = (uint64_t)SB * 210u;
    const uint32_t ngroups = (rows + 15u) >> 4;
    const uint32_t nrounds = (ngroups + slots - 1u) / slots;     // rounds of `slots` row groups
    const uint32_t odd = sb & 1u;
    const int32_t poff = q6m_piece_offset(lane, odd);
    auto issue = [&](uint32_t round_block, q6m_regs &W) {
        uint32_t rg = round_block * slots + (active ? slot : 0u);
        rg = rg < ngroups ? rg : ngroups - 1u;
        q6m_issue(w, row_bytes, rg * 16u, rows, sb, lane, poff, W);
    };
    q6m_regs Wa, Wb;
    uint32_t rb = blockIdx.x;
    // ... and the first row group's weights; with RMSNorm in front only once every wave's request
    // for its activations is in the CU's memory queue (a short load queued behind other waves'
    // long ones waits for them, and every wave waits for every wave's activations there)
    if (NORM) {
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("s_barrier" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
    }
    issue(rb, Wa);

    // ---- everything the tail of a round needs, while the loads are on their way ----
    double *norm = reinterpret_cast<double *>(smem + kPart);
    uint8_t *wave_lds = smem + kPart + kNorm + (size_t)wave * kWave;
    uint8_t *dig = wave_lds + kQAreaBytes, *zero = dig + NC * kQ1DigBytes;
    const uint32_t r = lane & 15u, q = lane >> 4;
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
        // RMSNorm as the reference computes it: mean square and 1/sqrt in f64, then (f32)(x * inv) * gain
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            double ss = (double)v[c].x * (double)v[c].x;
            ss = fma((double)v[c].y, (double)v[c].y, ss);
            ss = fma((double)v[c].z, (double)v[c].z, ss);
            ss = fma((double)v[c].w, (double)v[c].w, ss);
            ss = lev_group_sum_f64<64>(ss);                    // lane 63 holds the wave's sum
            if (lane == 63u) norm[c * kQWaves + wave] = ss;
        }
        lev_barrier_lds();
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            // the waves of slot 0 cover the row once: lane k of every row of 16 lanes takes wave k's
            // sum, and the row adds them up (every lane ends with the total)
            const double mine = norm[c * kQWaves + r];
            const double tot = lev_group_sum_f64<16>(r < wpr ? mine : 0.0);
            const double a = fma(tot, rcols, (double)eps);
            double rs = __builtin_amdgcn_rsq(a);
            rs = rs * fma(-0.5 * a * rs, rs, 1.5);
            rs = rs * fma(-0.5 * a * rs, rs, 1.5);
#pragma unroll
            for (int k = 0; k < 4; ++k) v[c][k] = (float)((double)v[c][k] * rs) * gn[k];
        }
    }

    // ---- the wave's digit planes (and, at one column, its A operands) ----
    double ps[NC];                                             // 2^(e - 2): undoes the scaling and the 4 of the codes
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        uint32_t mb = 0u;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint32_t bits = __float_as_uint(v[c][k]) & 0x7FFFFFFFu;
            mb = bits > mb ? bits : mb;
        }
        mb = lev_wave_max_u32(mb);
        uint32_t ex = mb >> 23;                             // biased exponent: |x| < 2^(ex-126)
        const bool bad = ex == 255u;                        // NaN or infinity in the superblock
        ex = ex < 30u ? 30u : (ex > 254u ? 254u : ex);      // keeps both powers of two normal numbers
        const float scale = __uint_as_float((283u - ex) << 23);   // 2^(156-ex): |x*scale| < 2^30
        ps[c] = !active ? 0.0 : bad ? (double)__builtin_nanf("") : __hiloint2double((int)((ex + 865u) << 20), 0);   // 2^(ex-158)
        uint32_t Y[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int X = (int)rintf(v[c][k] * scale);
            Y[k] = ((uint32_t)X + 0x00808080u) ^ 0x00808080u;   // bytes = balanced base-256 digits
        }
        const uint32_t t0 = __builtin_amdgcn_perm(Y[1], Y[0], 0x05010400u);
        const uint32_t t1 = __builtin_amdgcn_perm(Y[1], Y[0], 0x07030602u);
        const uint32_t t2 = __builtin_amdgcn_perm(Y[3], Y[2], 0x05010400u);
        const uint32_t t3 = __builtin_amdgcn_perm(Y[3], Y[2], 0x07030602u);
        const uint32_t dw[4] = {__builtin_amdgcn_perm(t2, t0, 0x05040100u), __builtin_amdgcn_perm(t2, t0, 0x07060302u),
                                __builtin_amdgcn_perm(t3, t1, 0x05040100u), __builtin_amdgcn_perm(t3, t1, 0x07060302u)};
        // group lane/4, plane p at +16p, the lane's four elements at +4*(lane%4)
        uint8_t *at = dig + c * kQ1DigBytes + (lane >> 2) * 64u + 4u * (lane & 3u);
#pragma unroll
        for (int p = 0; p < 4; ++p) *reinterpret_cast<uint32_t *>(at + 16 * p) = dw[p];
    }
    if (lane < kQ1ZeroBytes / 4u) reinterpret_cast<uint32_t *>(zero)[lane] = 0u;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    // lane (r, g) feeds A row r = 4*gs + p: plane p of group 8*hf + 2*jb (+ 4*nb + lh) when gs == g,
    // zeros otherwise
    const uint32_t hf = q >> 1, jb = q & 1u;
    const bool feeds = active && (r >> 2) == q;
    const uint8_t *ab = feeds ? dig + (8u * hf + 2u * jb) * 64u + 16u * (r & 3u) : zero;
    const uint32_t hs = feeds ? 64u : 0u, cs = feeds ? kQ1DigBytes : 0u;
    q6m_i4 A1[2][2];
    if (NC == 1) {
#pragma unroll
        for (int nb = 0; nb < 2; ++nb)
#pragma unroll
            for (int lh = 0; lh < 2; ++lh) A1[nb][lh] = *reinterpret_cast<const q6m_i4 *>(ab + (4 * nb + lh) * hs);
    }
    const q6m_lane L6(smem + kPart + kNorm, wave, lane, odd, kWave);
    // the operands are read back before the wait for the weights, not behind it
    __builtin_amdgcn_sched_barrier(0);

    top2 best{kTop2Floor, kTop2Floor, 0xFFFFFFFFu};
    auto finish = [&](const q6m_regs &W) {
        q6m_i4 B[2][2];
        int sc[2][2];
        uint32_t dbits;
        L6.operands(W, B, sc, dbits);
        const double d = (double)lev_f16_bits_to_f32(dbits);
        double val[NC];
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            int E[4] = {0, 0, 0, 0};
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) {
#pragma unroll
                for (int lh = 0; lh < 2; ++lh) {
                    const q6m_i4 A = NC == 1 ? A1[nb][lh]
                                             : *reinterpret_cast<const q6m_i4 *>(ab + c * cs + (4 * nb + lh) * hs);
                    const q6m_i4 D = __builtin_amdgcn_mfma_i32_16x16x64_i8(A, B[nb][lh], q6m_i4{0, 0, 0, 0}, 0, 0, 0);
                    // |D| <= 16*128*128 = 2^18, |sc| <= 2^7: four products per plane stay below 2^27
#pragma unroll
                    for (int p = 0; p < 4; ++p) {
                        E[p] += __mul24(D[p], sc[nb][lh]);
                        asm("" : "+v"(E[p]));   // one multiply-add per plane: keeps the sums from being regrouped
                    }
                }
            }
            const double hi = fma((double)E[3], 256.0, (double)E[2]);
            const double lo = fma((double)E[1], 256.0, (double)E[0]);
            const double dot = fma(hi, 65536.0, lo);
            val[c] = lev_row_sum_f64((ps[c] * d) * dot);
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
                if (stores && (uint32_t)c < ncol) {
                    const float out = (float)s;
                    *reinterpret_cast<__attribute__((address_space(1))) float *>(yp + (uint64_t)c * rows * 4u) = out;
                    if (NC == 1) {
                        // running top two of the rows this lane finishes (rows ascend, so a tie keeps
                        // the earlier, lower index)
                        if (out > best.best) {
                            best.second = best.best;
                            best.best = out;
                            best.idx = orow;
                        } else if (out > best.second) {
                            best.second = out;
                        }
                    }
                }
            }
        }
        pw ^= kQWaves * 16u * 8u * NC;                         // the other half of `part` next round
        pr ^= kQWaves * 16u * 8u * NC;
        orow += orow_step;
        yp += (uint64_t)orow_step * 4u;
        stores = writer && orow < rows ? 1u : 0u;
    };
    // Unconditional (clamped) prefetch, one round ahead (a branch around the loads would make the
    // compiler wait for them before the current group is multiplied).
    // (The scheduling barriers keep the requests where they are written: sunk below the products
    // of the round in hand they would no longer run ahead of anything.)
    while (true) {
        uint32_t next = rb + gridDim.x;
        __builtin_amdgcn_sched_barrier(0);
        issue(next < nrounds ? next : rb, Wb);
        __builtin_amdgcn_sched_barrier(0);
        finish(Wa);
        if (next >= nrounds) break;
        rb = next;
        next = rb + gridDim.x;
        __builtin_amdgcn_sched_barrier(0);
        issue(next < nrounds ? next : rb, Wa);
        __builtin_amdgcn_sched_barrier(0);
        finish(Wb);
        if (next >= nrounds) break;
        rb = next;
    }
    if (NC == 1 && partials) q6m_greedy_token(best, slots, partials, tickets, out_idx, out_margin);
}

// ---------------------------------------------------------------------------
// The same weight stream on int8 activations (q6k.q8.matvec, emit_q6k_q8,
// lev-forge/src/q8.rs:330-447; oracle matvec_q6k_q8_f64, lev-cpu/src/lib.rs:333-337):
// xq int8 [ncol][cols], xs (d, s) pairs per 32 activations.  A row 4*gs + c of an MFMA
// holds the codes of column c (of a chunk of four) for the k-slots lane group gs
// supplies, so one MFMA gives a lane the exact sums 4*(q-32)*xq over one 16-weight group
// for four columns; the two halves of a 32-activation block take their int8 scales in
// integers, then the block's activation scale in f32:
//   y[c] += d * sum_blocks dx[c][block] * (sc_a * D_a[c] + sc_b * D_b[c]) / 4.
// (The -32 of the codes is inside the operand, so the s of the pairs is not used.)
// LDS: codes [NC][cols] as they come, dx [cols/32][NC] f32 (x 1/4), partial sums
// [pb][16 waves][16 rows][NC] f32, the turn-round areas.
// ---------------------------------------------------------------------------
template <int NC>
struct q6m_q8_lds {
    static __host__ __device__ size_t total(uint32_t cols, uint32_t pb) {
        return (size_t)NC * cols + kQZeroBytes + (size_t)(cols >> 5) * NC * 4u +
               (size_t)pb * kQWaves * 16u * NC * 4u + (size_t)kQWaves * kQAreaBytes;
    }
};

// NC: columns staged (4, 8 or 16; >= ncol).
// NC: columns staged (4, 8 or 16; >= ncol).  DEPTH: tasks in flight per wave (3; 2 at sixteen
// columns, whose accumulators leave no registers for a third).
template <int NC, int DEPTH>
__global__ void __launch_bounds__(kQThreads)
q6_k_mfma_gemv_q8(const uint8_t *__restrict__ w, const uint32_t *__restrict__ xq, const float *__restrict__ xs,
                  float *__restrict__ y, uint32_t cols, uint32_t rows, uint32_t ncol, uint32_t S, uint32_t pb) {
    constexpr int NCH = NC / 4;
    constexpr uint32_t kLogNC = NC == 16 ? 4u : NC == 8 ? 3u : 2u;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const uint32_t SB = cols >> 8, nblk = cols >> 5;
    uint8_t *dig = smem;
    uint8_t *zero = smem + (size_t)NC * cols;
    float *dxs = reinterpret_cast<float *>(zero + kQZeroBytes);
    float *part = dxs + (size_t)nblk * NC;
    uint8_t *area_all = reinterpret_cast<uint8_t *>(part + (size_t)pb * kQWaves * 16u * NC);

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t r = lane & 15u, g = lane >> 4;
    const uint64_t row_bytes = (uint64_t)SB * 210u;
    const uint32_t ngroups = (rows + 15u) >> 4;
    const uint32_t slots = kQWaves / S;
    const uint32_t slot = wave / S, kpart = wave % S;
    const uint32_t tpr = (SB + S - 1u) / S;
    const uint32_t wgrounds = (ngroups + slots - 1u) / slots;
    const uint32_t nrounds = (wgrounds - blockIdx.x + gridDim.x - 1u) / gridDim.x;
    const uint32_t ntasks = nrounds * tpr;
    struct cursor {
        uint32_t k, rd, t;
    };
    auto advance = [&](cursor &c) {
        ++c.k;
        if (++c.t == tpr) {
            c.t = 0;
            ++c.rd;
        }
    };
    const uint32_t odd = kpart & 1u;
    const int32_t poff = q6m_piece_offset(lane, odd), poff_even = q6m_piece_offset(lane, 0u);
    auto group_of = [&](uint32_t rd, uint32_t sl) { return (rd * gridDim.x + blockIdx.x) * slots + sl; };
    auto issue = [&](cursor &c, q6m_regs &W) {
        const uint32_t sbw = kpart + S * c.t;
        const bool real = c.k < ntasks && sbw < SB;
        q6m_issue(w, row_bytes, real ? group_of(c.rd, slot) * 16u : 0u, rows, real ? sbw : 0u, lane,
                  real ? poff : poff_even, W);
        advance(c);
    };
    cursor ci{0u, 0u, 0u}, cc{0u, 0u, 0u};
    q6m_regs W0, W1, W2;

    // ---- stage the activations: the codes as they come, the block scales transposed ----
    if (tid < kQZeroBytes / 4u) reinterpret_cast<uint32_t *>(zero)[tid] = 0u;
    {
        const lev_u32x4 *src = reinterpret_cast<const lev_u32x4 *>(xq);
        lev_u32x4 *dst = reinterpret_cast<lev_u32x4 *>(dig);
        const uint32_t n16 = ncol * (cols >> 4);
        for (uint32_t i = tid; i < n16; i += kQThreads) dst[i] = src[i];
        // columns of the layout beyond ncol: zero codes and scales (their outputs are never stored)
        for (uint32_t i = n16 + tid; i < (uint32_t)NC * (cols >> 4); i += kQThreads) dst[i] = lev_u32x4{0u, 0u, 0u, 0u};
        for (uint32_t i = tid; i < nblk * NC; i += kQThreads) {
            const uint32_t c = i & (NC - 1u), b = i >> kLogNC;
            // a quarter of the activation scale: the codes in the operand are 4*(q - 32)
            dxs[i] = c < ncol ? 0.25f * xs[((uint64_t)c * nblk + b) * 2u] : 0.f;
        }
    }
    lev_barrier_lds();
    issue(ci, W0);

    // ---- stream the weights ----
    const uint32_t hf = g >> 1, jb = g & 1u;
    const bool feeds = (r >> 2) == g;
    const q6m_lane L6(area_all, wave, lane, odd);
    float yacc[NCH][4];
#pragma unroll
    for (int ch = 0; ch < NCH; ++ch)
#pragma unroll
        for (int i = 0; i < 4; ++i) yacc[ch][i] = 0.f;

    uint32_t parity = 0;
    auto compute = [&](cursor &c, const q6m_regs &W) {
        const uint32_t rd = c.rd, t = c.t;
        const uint32_t sbw = kpart + S * t;
        const bool live = sbw < SB;
        const uint32_t sb = live ? sbw : SB - 1u;
        q6m_i4 B[2][2];
        int sc[2][2];
        uint32_t dbits;
        L6.operands(W, B, sc, dbits);
        const float d = live ? lev_f16_bits_to_f32(dbits) : 0.f;
        // lane (r, g) feeds A row r = 4*gs + c: column 4*ch + r%4, the 16 codes of weight group
        // 16*sb + 8*hf + 2*jb (+ 4*nb + lh) when gs == g, zeros otherwise
        const uint32_t aoff = (r & 3u) * cols + (16u * sb + 8u * hf + 2u * jb) * 16u;
        const uint32_t blk0 = 8u * sb + 4u * hf + jb;   // 32-activation block of nb = 0; nb = 1: + 2
#pragma unroll
        for (int ch = 0; ch < NCH; ++ch) {
            const uint8_t *ab = feeds ? dig + (size_t)(4 * ch) * cols + aoff : zero;
            float ysb[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) {
                const q6m_i4 A0 = *reinterpret_cast<const q6m_i4 *>(ab + (4 * nb) * 16);
                const q6m_i4 A1 = *reinterpret_cast<const q6m_i4 *>(ab + (4 * nb + 1) * 16);
                const lev_f32x4 dx = *reinterpret_cast<const lev_f32x4 *>(dxs + (size_t)(blk0 + 2u * nb) * NC + 4 * ch);
                const q6m_i4 D0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(A0, B[nb][0], q6m_i4{0, 0, 0, 0}, 0, 0, 0);
                const q6m_i4 D1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(A1, B[nb][1], q6m_i4{0, 0, 0, 0}, 0, 0, 0);
                // |D| <= 16*128*127 < 2^18, |sc| <= 2^7: the sum of the two halves fits 32 bits
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    int E = __mul24(D0[i], sc[nb][0]);
                    E += __mul24(D1[i], sc[nb][1]);
                    ysb[i] = fmaf((float)E, dx[i], ysb[i]);
                }
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) yacc[ch][i] = fmaf(d, ysb[i], yacc[ch][i]);
        }

        if (t + 1u == tpr) {   // workgroup-uniform: the round ends
            float *pp = part + parity * (kQWaves * 16u * NC);
            parity ^= pb - 1u;
            // the four lane groups' shares of a row meet; lane group g keeps column 4*ch + g
#pragma unroll
            for (int ch = 0; ch < NCH; ++ch) {
                float mine = 0.f;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float v = yacc[ch][i];
                    v += __shfl_xor(v, 16);
                    v += __shfl_xor(v, 32);
                    mine = g == (uint32_t)i ? v : mine;
                    yacc[ch][i] = 0.f;
                }
                pp[(wave * 16u + r) * NC + 4u * (uint32_t)ch + g] = mine;
            }
            lev_barrier_lds();
            for (uint32_t i = tid; i < slots * 16u * NC; i += kQThreads) {
                const uint32_t rr = i & 15u, col = (i >> 4) & (NC - 1u), sl = i >> (4u + kLogNC);
                const uint32_t row = group_of(rd, sl) * 16u + rr;
                float sum = 0.f;
                for (uint32_t k = 0; k < S; ++k) sum += pp[((sl * S + k) * 16u + rr) * NC + col];
                if (col < ncol && row < rows) y[(uint64_t)col * rows + row] = sum;
            }
            if (pb == 1u) lev_barrier_lds();   // the one buffer is written again by the next round
        }
        advance(c);
    };

    issue(ci, W1);
    if (DEPTH > 2) issue(ci, W2);
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
        if (DEPTH > 2) {
            compute(cc, W2);
            __builtin_amdgcn_sched_barrier(0);
            issue(ci, W2);
            __builtin_amdgcn_sched_barrier(0);
            if (cc.k >= ntasks) break;
        }
    }
}

// ---------------------------------------------------------------------------
// Int8 activations, up to eight columns, rows of at most sixteen superblocks: a wave per
// superblock COLUMN of the matrix, as q6_k_mfma_gemv_one.  The A operands are the activation
// codes as they lie in memory (16 consecutive codes of one column), so a lane loads the ones of
// its wave's superblock straight into registers, with the quarter activation scales of its
// blocks beside them: nothing is staged in LDS but the turn-round of the weights and the
// partial sums of a round.
// LDS: part [2][16 waves][16 rows][NC] f32 | per wave: the turn-round area.
// ---------------------------------------------------------------------------
__host__ __device__ constexpr uint32_t q6m_q8_one_part_bytes(uint32_t nc) { return 2u * kQWaves * 16u * 4u * nc; }
__host__ __device__ constexpr size_t q6m_q8_one_lds(uint32_t nc) {
    return q6m_q8_one_part_bytes(nc) + (size_t)kQWaves * kQAreaBytes;
}

// NC: columns staged (4 or 8; >= ncol).
template <int NC>
__global__ void __launch_bounds__(kQThreads)
q6_k_mfma_gemv_q8_one(const uint8_t *__restrict__ w, const uint32_t *__restrict__ xq, const float *__restrict__ xs,
                      float *__restrict__ y, uint32_t cols, uint32_t rows, uint32_t ncol, uint32_t wpr, uint32_t slots,
                      uint64_t slot_of_wave, uint64_t pos_of_wave) {
    constexpr int NCH = NC / 4;
    constexpr uint32_t kPart = q6m_q8_one_part_bytes(NC);
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const uint32_t slot = (uint32_t)(slot_of_wave >> (4u * wave)) & 15u;   // idle waves: slot >= slots
    const uint32_t sb = (uint32_t)(pos_of_wave >> (4u * wave)) & 15u;      // the wave's superblock column
    const uint32_t SB = cols >> 8, nblk = cols >> 5;
    const uint32_t r = lane & 15u, q = lane >> 4;
    const uint32_t hf = q >> 1, jb = q & 1u;
    const bool active = slot < slots;

    // the wave's activations first: lane (r, g) feeds A row r = 4*gs + c, i.e. column 4*ch + r%4,
    // the 16 codes of weight group 16*sb + 8*hf + 2*jb (+ 4*nb + lh), when gs == g, zeros
    // otherwise (columns of the layout beyond ncol repeat the last one and are never stored)
    q6m_i4 A[NCH][2][2];
    float dx[NCH][2][4];   // a quarter of the activation scale (the codes in the operand are 4*(q - 32)) of block nb, column 4*ch + i
    const uint32_t blk0 = 8u * sb + 4u * hf + jb;   // 32-activation block of nb = 0; nb = 1: + 2
#pragma unroll
    for (int ch = 0; ch < NCH; ++ch) {
        const uint32_t ca = 4u * (uint32_t)ch + (r & 3u);
        const uint8_t *xa = reinterpret_cast<const uint8_t *>(xq) + (uint64_t)(ca < ncol ? ca : ncol - 1u) * cols +
                            256u * sb + (8u * hf + 2u * jb) * 16u;
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) {
#pragma unroll
            for (int lh = 0; lh < 2; ++lh) A[ch][nb][lh] = *reinterpret_cast<const q6m_i4 *>(xa + (4 * nb + lh) * 16);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint32_t ci = 4u * (uint32_t)ch + (uint32_t)i;
                dx[ch][nb][i] = xs[((uint64_t)(ci < ncol ? ci : ncol - 1u) * nblk + blk0 + 2u * (uint32_t)nb) * 2u];
            }
        }
    }
    // ... the first row group's weights right behind them
    const uint64_t row_bytes = (uint64_t)SB * 210u;
    const uint32_t ngroups = (rows + 15u) >> 4;
    const uint32_t nrounds = (ngroups + slots - 1u) / slots;     // rounds of `slots` row groups
    const uint32_t odd = sb & 1u;
    const int32_t poff = q6m_piece_offset(lane, odd);
    auto issue = [&](uint32_t round_block, q6m_regs &W) {
        uint32_t rg = round_block * slots + (active ? slot : 0u);
        rg = rg < ngroups ? rg : ngroups - 1u;
        q6m_issue(w, row_bytes, rg * 16u, rows, sb, lane, poff, W);
    };
    q6m_regs Wa, Wb;
    uint32_t rb = blockIdx.x;
    issue(rb, Wa);

    // ---- everything the tail of a round needs, while the loads are on their way ----
    uint32_t pw = ((wave * 16u + r) * NC + q) * 4u;              // lane (r, q): row r, column q (+ 4 per chunk)
    uint32_t pr = ((((wave < slots ? wave : 0u) * wpr) * 16u + r) * NC + q) * 4u;
    uint32_t orow = (rb * slots + wave) * 16u + r;
    const uint32_t orow_step = gridDim.x * slots * 16u;
    const bool writer = wave < slots;
    uint32_t stores = writer && orow < rows ? 1u : 0u;
    uint64_t yp = reinterpret_cast<uint64_t>(y + (uint64_t)q * rows + orow);
    lev_pin(pw);
    lev_pin(pr);
    lev_pin(stores);
    lev_pin(yp);
    const bool feeds = active && (r >> 2) == q;
#pragma unroll
    for (int ch = 0; ch < NCH; ++ch)
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) {
#pragma unroll
            for (int lh = 0; lh < 2; ++lh) A[ch][nb][lh] = feeds ? A[ch][nb][lh] : q6m_i4{0, 0, 0, 0};
#pragma unroll
            for (int i = 0; i < 4; ++i) dx[ch][nb][i] *= active ? 0.25f : 0.f;
        }
    const q6m_lane L6(smem + kPart, wave, lane, odd);
    __builtin_amdgcn_sched_barrier(0);

    auto finish = [&](const q6m_regs &W) {
        q6m_i4 B[2][2];
        int sc[2][2];
        uint32_t dbits;
        L6.operands(W, B, sc, dbits);
        const float d = lev_f16_bits_to_f32(dbits);
#pragma unroll
        for (int ch = 0; ch < NCH; ++ch) {
            float v[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) {
                const q6m_i4 D0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[ch][nb][0], B[nb][0], q6m_i4{0, 0, 0, 0}, 0, 0, 0);
                const q6m_i4 D1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[ch][nb][1], B[nb][1], q6m_i4{0, 0, 0, 0}, 0, 0, 0);
                // |D| <= 16*128*127 < 2^18, |sc| <= 2^7: the sum of the two halves fits 32 bits
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    int E = __mul24(D0[i], sc[nb][0]);
                    E += __mul24(D1[i], sc[nb][1]);
                    v[i] = fmaf((float)E, dx[ch][nb][i], v[i]);
                }
            }
            // the four lane groups' shares of a row meet, lane group g keeping column 4*ch + g
            *reinterpret_cast<float *>(smem + pw + 16 * ch) = d * lev_lanegroup_sums4(v);
        }
        lev_barrier_lds();
        if (wave < slots) {
            const float *pp = reinterpret_cast<const float *>(smem + pr);
#pragma unroll
            for (int ch = 0; ch < NCH; ++ch) {
                // the slot's waves in order, four chains added at the end (sixteen reads in flight)
                float s4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int k = 0; k < kQWaves; ++k) {
                    const float pk = pp[k * 16 * NC + 4 * ch];
                    s4[k & 3] += (uint32_t)k < wpr ? pk : 0.f;
                }
                const float s = (s4[0] + s4[1]) + (s4[2] + s4[3]);
                if (stores && 4u * (uint32_t)ch + q < ncol)
                    *reinterpret_cast<__attribute__((address_space(1))) float *>(yp + (uint64_t)(4 * ch) * rows * 4u) = s;
            }
        }
        pw ^= kQWaves * 16u * 4u * NC;                         // the other half of `part` next round
        pr ^= kQWaves * 16u * 4u * NC;
        orow += orow_step;
        yp += (uint64_t)orow_step * 4u;
        stores = writer && orow < rows ? 1u : 0u;
    };
    // Unconditional (clamped) prefetch, one round ahead; the scheduling barriers keep the requests
    // where they are written.
    while (true) {
        uint32_t next = rb + gridDim.x;
        __builtin_amdgcn_sched_barrier(0);
        issue(next < nrounds ? next : rb, Wb);
        __builtin_amdgcn_sched_barrier(0);
        finish(Wa);
        if (next >= nrounds) break;
        rb = next;
        next = rb + gridDim.x;
        __builtin_amdgcn_sched_barrier(0);
        issue(next < nrounds ? next : rb, Wa);
        __builtin_amdgcn_sched_barrier(0);
        finish(Wb);
        if (next >= nrounds) break;
        rb = next;
    }
}

size_t q6m_lds_limit(const lev_ctx *ctx) {
    return ctx->props.sharedMemPerBlockOptin > ctx->props.sharedMemPerBlock ? ctx->props.sharedMemPerBlockOptin
                                                                            : ctx->props.sharedMemPerBlock;
}

size_t q6m_lds_bytes(uint32_t cols, uint32_t nc, uint32_t pb) {
    switch (nc) {
    case 8: return q6m_lds<8>::total(cols, pb);
    case 4: return q6m_lds<4>::total(cols, pb);
    case 2: return q6m_lds<2>::total(cols, pb);
    default: return q6m_lds<1>::total(cols, pb);
    }
}

// Waves per row group.  The busiest workgroup runs ceil(rounds / grid) rounds of SB/S tasks:
// the smallest S that makes that product smallest (fewer partial sums to add up).
uint32_t q6m_waves_per_group(const lev_ctx *ctx, uint32_t cols, uint32_t rows) {
    // LEV_Q6_MFMA_WAVES (experiments): only the values the kernel is built for; anything else is ignored
    static const int forced = [] {
        const char *env = getenv("LEV_Q6_MFMA_WAVES");
        const int v = env ? atoi(env) : 0;
        return v == 2 || v == 4 || v == 8 || v == 16 ? v : 0;
    }();
    if (forced) return (uint32_t)forced;
    const uint32_t SB = cols >> 8, ngroups = (rows + 15u) / 16u, cus = (uint32_t)ctx->num_cus;
    uint32_t best = 2, best_cost = 0xFFFFFFFFu;
    for (uint32_t s = 2; s <= (uint32_t)kQWaves; s <<= 1) {   // even: a wave's superblocks share their parity
        const uint32_t slots = kQWaves / s, wgrounds = (ngroups + slots - 1u) / slots;
        const uint32_t cost = ((wgrounds + cus - 1u) / cus) * ((SB + s - 1u) / s);
        if (cost < best_cost) best_cost = cost, best = s;
    }
    return best;
}

template <int NC>
hipError_t q6m_launch(lev_ctx *ctx, const uint8_t *w, const float *x, const float *gain, float eps, float *y,
                      uint32_t cols, uint32_t rows, uint32_t ncol, uint32_t waves, lev_f32x4 *partials,
                      uint32_t *d_argmax, float *d_margin) {
    const uint32_t pb = q6m_lds_bytes(cols, NC, 2u) <= q6m_lds_limit(ctx) ? 2u : 1u;
    const size_t lds = q6m_lds_bytes(cols, NC, pb);
    static size_t configured = 0;   // per instantiation: raise the dynamic LDS limit once per size
    if (lds > 48 * 1024 && lds > configured) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&q6_k_mfma_gemv<NC>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        configured = lds;
    }
    const uint32_t S = waves ? waves : q6m_waves_per_group(ctx, cols, rows);
    const uint32_t slots = kQWaves / S, ngroups = (rows + 15u) / 16u;
    const uint32_t wgrounds = (ngroups + slots - 1u) / slots;
    uint32_t blocks = wgrounds < (uint32_t)ctx->num_cus ? wgrounds : (uint32_t)ctx->num_cus;
    if (partials && blocks > lev_ctx::kArgmaxPartials) blocks = lev_ctx::kArgmaxPartials;
    uint32_t *tickets = partials ? reinterpret_cast<uint32_t *>(ctx->d_flag) + lev_ctx::kArgmaxTicketWord : nullptr;
    hipLaunchKernelGGL((q6_k_mfma_gemv<NC>), dim3(blocks), dim3(kQThreads), lds, ctx->stream, w, x, gain, eps,
                       y, cols, rows, ncol, S, pb, 1.0 / (double)cols, partials, tickets, d_argmax, d_margin);
    return hipGetLastError();
}

template <int NC, bool NORM>
hipError_t q6m_one_launch(lev_ctx *ctx, const uint8_t *w, const float *x, const float *gain, float eps, float *y,
                          uint32_t cols, uint32_t rows, uint32_t ncol, lev_f32x4 *partials, uint32_t *d_argmax,
                          float *d_margin) {
    const uint32_t wpr = cols >> 8, slots = (uint32_t)kQWaves / wpr;
    const uint32_t ngroups = (rows + 15u) / 16u;
    const uint32_t nrounds = (ngroups + slots - 1u) / slots;
    uint64_t slot_of_wave, pos_of_wave;
    lev_wave_tables(wpr, &slot_of_wave, &pos_of_wave);
    constexpr size_t lds = q6m_one_lds(NC);
    static bool configured = false;   // per instantiation: raise the dynamic LDS limit once
    if (!configured) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&q6_k_mfma_gemv_one<NC, NORM>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        configured = true;
    }
    if (NC != 1) partials = nullptr;
    uint32_t blocks = nrounds < (uint32_t)ctx->num_cus ? nrounds : (uint32_t)ctx->num_cus;
    if (partials && blocks > lev_ctx::kArgmaxPartials) blocks = lev_ctx::kArgmaxPartials;
    uint32_t *tickets = partials ? reinterpret_cast<uint32_t *>(ctx->d_flag) + lev_ctx::kArgmaxTicketWord : nullptr;
    hipLaunchKernelGGL((q6_k_mfma_gemv_one<NC, NORM>), dim3(blocks), dim3(kQThreads), lds, ctx->stream, w, x, gain,
                       eps, y, cols, rows, ncol, wpr, slots, slot_of_wave, pos_of_wave, 1.0 / (double)cols, partials,
                       tickets, d_argmax, d_margin);
    return hipGetLastError();
}

template <int NC>
hipError_t q6m_one_launch_nc(lev_ctx *ctx, const uint8_t *w, const float *x, const float *gain, float eps, float *y,
                             uint32_t cols, uint32_t rows, uint32_t ncol, lev_f32x4 *partials, uint32_t *d_argmax,
                             float *d_margin) {
    if (gain) return q6m_one_launch<NC, true>(ctx, w, x, gain, eps, y, cols, rows, ncol, partials, d_argmax, d_margin);
    return q6m_one_launch<NC, false>(ctx, w, x, gain, eps, y, cols, rows, ncol, partials, d_argmax, d_margin);
}

}  // namespace

// Columns one launch of the matrix-core kernel can take for this in_dim (0: not usable).
uint32_t lev_q6_k_mfma_cols(const lev_ctx *ctx, uint32_t in_dim) {
    if (in_dim % 256u != 0u || in_dim == 0u) return 0;
    uint32_t nc = 8;
    const size_t limit = q6m_lds_limit(ctx);
    while (nc >= 1u && ((uint64_t)nc * in_dim > 32768u || q6m_lds_bytes(in_dim, nc, 1u) > limit)) nc >>= 1;
    return nc;
}

// The built-in number of waves per row group for a shape.
uint32_t lev_q6_k_mfma_waves(const lev_ctx *ctx, uint32_t in_dim, uint32_t rows) {
    return q6m_waves_per_group(ctx, in_dim, rows);
}

// ncol <= lev_q6_k_mfma_cols(ctx, in_dim); w 2-byte, x and gain 16-byte aligned.  waves: 2, 4,
// 8 or 16 waves per row group, 0 for the built-in choice.  d_argmax / d_margin (ncol == 1
// only, both may be NULL): the greedy token of the column, merged by the last workgroup to
// finish from one top-two record per workgroup in `partials` (lev_ctx::kArgmaxPartials
// records).
hipError_t lev_q6_k_mfma_gemv_launch(lev_ctx *ctx, const uint8_t *w, const float *x, const float *gain,
                                     float eps, float *y, uint32_t in_dim, uint32_t rows, uint32_t ncol,
                                     uint32_t waves, lev_f32x4 *partials, uint32_t *d_argmax, float *d_margin) {
    if (!d_argmax && !d_margin) partials = nullptr;
    if (waves != 2u && waves != 4u && waves != 8u && waves != 16u) waves = 0u;
    // one or two columns of at most sixteen superblocks, no number of waves per row group asked
    // for: a wave per superblock column (four columns measured 31.5 us at 32000 x 4096 either way:
    // a column costs its products and recombination again, and the several-column kernel stages
    // the planes once per workgroup)
    static const bool one_off = [] {
        const char *e = getenv("LEV_Q6K_ONE");   // LEV_Q6K_ONE=0: the several-column kernel at one column too, for comparison
        return e && e[0] == '0';
    }();
    if (ncol <= 2u && waves == 0u && !one_off && in_dim <= 4096u) {
        if (ncol > 1u) return q6m_one_launch_nc<2>(ctx, w, x, gain, eps, y, in_dim, rows, ncol, partials, d_argmax, d_margin);
        return q6m_one_launch_nc<1>(ctx, w, x, gain, eps, y, in_dim, rows, ncol, partials, d_argmax, d_margin);
    }
    if (ncol > 4) return q6m_launch<8>(ctx, w, x, gain, eps, y, in_dim, rows, ncol, waves, partials, d_argmax, d_margin);
    if (ncol > 2) return q6m_launch<4>(ctx, w, x, gain, eps, y, in_dim, rows, ncol, waves, partials, d_argmax, d_margin);
    if (ncol > 1) return q6m_launch<2>(ctx, w, x, gain, eps, y, in_dim, rows, ncol, waves, partials, d_argmax, d_margin);
    return q6m_launch<1>(ctx, w, x, gain, eps, y, in_dim, rows, ncol, waves, partials, d_argmax, d_margin);
}

namespace {
size_t q6m_q8_lds_bytes(uint32_t cols, uint32_t nc, uint32_t pb) {
    return nc > 8u ? q6m_q8_lds<16>::total(cols, pb) : nc > 4u ? q6m_q8_lds<8>::total(cols, pb)
                                                                 : q6m_q8_lds<4>::total(cols, pb);
}

template <int NC>
hipError_t q6m_q8_launch(lev_ctx *ctx, const uint8_t *w, const uint32_t *xq, const float *xs, float *y,
                         uint32_t cols, uint32_t rows, uint32_t ncol, uint32_t waves) {
    const uint32_t pb = q6m_q8_lds_bytes(cols, NC, 2u) <= q6m_lds_limit(ctx) ? 2u : 1u;
    const size_t lds = q6m_q8_lds_bytes(cols, NC, pb);
    static size_t configured = 0;   // per instantiation: raise the dynamic LDS limit once per size
    if (lds > 48 * 1024 && lds > configured) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&q6_k_mfma_gemv_q8<NC, (NC > 8 ? 2 : 3)>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        configured = lds;
    }
    const uint32_t S = waves ? waves : q6m_waves_per_group(ctx, cols, rows);
    const uint32_t slots = kQWaves / S, ngroups = (rows + 15u) / 16u;
    const uint32_t wgrounds = (ngroups + slots - 1u) / slots;
    const uint32_t blocks = wgrounds < (uint32_t)ctx->num_cus ? wgrounds : (uint32_t)ctx->num_cus;
    hipLaunchKernelGGL((q6_k_mfma_gemv_q8<NC, (NC > 8 ? 2 : 3)>), dim3(blocks), dim3(kQThreads), lds, ctx->stream, w, xq, xs, y,
                       cols, rows, ncol, S, pb);
    return hipGetLastError();
}
}  // namespace

// Columns one launch of the int8-activation matrix-core kernel can take for this in_dim (0: not usable).
uint32_t lev_q6_k_mfma_q8_cols(const lev_ctx *ctx, uint32_t in_dim) {
    if (in_dim % 256u != 0u || in_dim == 0u) return 0;
    const size_t limit = q6m_lds_limit(ctx);
    for (uint32_t nc = 16; nc >= 4u; nc >>= 1)
        if (q6m_q8_lds_bytes(in_dim, nc, 1u) <= limit) return nc;
    return 0;
}

namespace {
template <int NC>
hipError_t q6m_q8_one_launch(lev_ctx *ctx, const uint8_t *w, const uint32_t *xq, const float *xs, float *y,
                             uint32_t cols, uint32_t rows, uint32_t ncol) {
    const uint32_t wpr = cols >> 8, slots = (uint32_t)kQWaves / wpr;
    const uint32_t ngroups = (rows + 15u) / 16u;
    const uint32_t nrounds = (ngroups + slots - 1u) / slots;
    uint64_t slot_of_wave, pos_of_wave;
    lev_wave_tables(wpr, &slot_of_wave, &pos_of_wave);
    constexpr size_t lds = q6m_q8_one_lds(NC);
    static bool configured = false;   // per instantiation: raise the dynamic LDS limit once
    if (!configured) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&q6_k_mfma_gemv_q8_one<NC>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        configured = true;
    }
    const uint32_t blocks = nrounds < (uint32_t)ctx->num_cus ? nrounds : (uint32_t)ctx->num_cus;
    hipLaunchKernelGGL((q6_k_mfma_gemv_q8_one<NC>), dim3(blocks), dim3(kQThreads), lds, ctx->stream, w, xq, xs, y,
                       cols, rows, ncol, wpr, slots, slot_of_wave, pos_of_wave);
    return hipGetLastError();
}
}  // namespace

// ncol <= lev_q6_k_mfma_q8_cols(ctx, in_dim); w 2-byte, xq 16-byte, xs 8-byte aligned.
hipError_t lev_q6_k_mfma_gemv_q8_launch(lev_ctx *ctx, const uint8_t *w, const uint32_t *xq, const float *xs,
                                        float *y, uint32_t in_dim, uint32_t rows, uint32_t ncol, uint32_t waves) {
    if (waves != 2u && waves != 4u && waves != 8u && waves != 16u) waves = 0u;
    // up to eight columns of at most sixteen superblocks, no number of waves per row group asked
    // for: a wave per superblock column
    static const bool one_off = [] {
        const char *e = getenv("LEV_Q6K_ONE");
        return e && e[0] == '0';
    }();
    if (ncol <= 8u && waves == 0u && !one_off && in_dim <= 4096u) {
        if (ncol > 4u) return q6m_q8_one_launch<8>(ctx, w, xq, xs, y, in_dim, rows, ncol);
        return q6m_q8_one_launch<4>(ctx, w, xq, xs, y, in_dim, rows, ncol);
    }
    if (ncol > 8) return q6m_q8_launch<16>(ctx, w, xq, xs, y, in_dim, rows, ncol, waves);
    if (ncol > 4) return q6m_q8_launch<8>(ctx, w, xq, xs, y, in_dim, rows, ncol, waves);
    return q6m_q8_launch<4>(ctx, w, xq, xs, y, in_dim, rows, ncol, waves);
}

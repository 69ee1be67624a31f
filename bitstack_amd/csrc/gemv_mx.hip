// One- and two-token packed-sign GEMV on the block-scaled MFMA of gfx950
// (v_mfma_scale_f32_16x16x128_f8f6f4): signs as the fp4 operand, Z = vt o x as fp6.
//
//   y[m] = sum_i sum_r u_i[m, r] * ( sum_n s_i[m, n] * Z_i[r, n] ),   Z_i[r, n] = vt_i[r, n] * x[n]
//
// Same contraction as gemv_kernel (D[r, m] += Z[r, n] S[m, n] on the matrix cores, 16 MACs per
// sign bit), but one MFMA now takes K = 128 columns and both operands come cheap:
//
// ---- the sign operand: one VALU instruction per EIGHT signs -----------------------------
// An fp4 (e2m1) operand register holds eight 4-bit codes.  A lane keeps its 16 bytes of signs
// (128 columns of one row) as loaded; MFMA number q = 3..0 of those columns uses bit q of every
// nibble, so its four operand registers are `word & (0x11111111 << q)`, nothing else:
//     q = 3   the fp4 sign bit, merged with the code of 1.0: (w & 0x88888888) | 0x22222222 = -+1
//             (bit set = code -1.0 although it means +1: Z enters negated for these columns)
//     q = 2   code 0100 = 2.0 or 0           B scale 1   value 1 + s
//     q = 1   code 0010 = 1.0 or 0           B scale 2   value 1 + s
//     q = 0   code 0001 = 0.5 or 0           B scale 4   value 1 + s
// so for q < 3 the MFMA accumulates sum (1 + s) z = sum z + sum s z.  The first sum does not
// depend on the row: the wave that produced the Z operand adds it up with one extra MFMA per
// term against the constant operand 1.0, and the shares are exchanged through LDS at flush time
// and subtracted (exactly: the same quantised z on both sides).
// Nibble e of word p of a lane in lane group g is column 128 g + 8 (4 p + e / 2) + (e odd ? 3 - q
// : 7 - q) of the lane's 512-column half unit: the Z operand is produced in that order.
//
// ---- the Z operand: three fp6 terms with block scales -----------------------------------
// z = vt * x is formed in fp16 (as gemv_kernel does), then split per (rank, 32 columns of one
// MFMA lane) into z = t1 2^e1 + t2 2^(e1-4) + t3 2^(e1-8) + rest with t_k in e2m3, by the
// hardware conversion v_cvt_scalef32_pk32_fp6_f16 (32 halves -> 32 packed fp6, round to nearest)
// and its inverse: t1 = cvt(z / 2^e1), r1 = z - t1 2^e1 (exact in fp16), t2 = cvt(r1 / 2^(e1-4)),
// ...  e1 puts the block maximum in [3.75, 7.5] (the top of e2m3), so |r1| <= 2^e1 / 4,
// |r2| <= 2^e1 / 128, |rest| <= 2^(e1-12): under 7e-5 of the block maximum, a fifth of the fp16
// rounding z already carries.  The three terms are three MFMAs into one accumulator, their
// scales the three low bytes of one E8M0 scale register.
//
// A unit is (block, row tile of 8 * R * 16 rows, 1024 columns) - with two tokens 512 columns of
// both, so that the operand images of a unit stay the same size: both 64-byte halves of every
// 128-byte line of sign bytes are requested back to back by the same lane (one unit apart with two tokens).  Z for the next unit
// is produced by all 512 threads while the current one is multiplied: wave w loads four ranks
// of one 512-column half (every vt value once per workgroup, coalesced), forms the products and
// passes them through a transpose in LDS to the lanes that convert them, 32 values each.
//
// What bounds it (counters and switch-off builds on an MI355X): the scaled MFMA occupies its SIMD
// for 16 + 4 cycles (matrix pipe + scale load) and VALU work of the other wave on the SIMD does
// not run underneath it, so a unit costs the SUM of 3 MFMAs (60 cycles) and 4 ANDs (16 cycles)
// per 16 x 128 signs plus the production of Z (about a third of that at 512 rows per workgroup):
// about 4.5 TB/s of sign bytes over 256 CUs, before the fill and drain of the pipeline.
#include "gemv_shared.h"

#include <type_traits>
#include <utility>

namespace {

typedef int v8i_t __attribute__((ext_vector_type(8)));
typedef unsigned v6u_t __attribute__((ext_vector_type(6)));
typedef _Float16 half32_t __attribute__((ext_vector_type(32)));
typedef uint16_t ushort2_t __attribute__((ext_vector_type(2)));
typedef uint32_t v16u_t __attribute__((ext_vector_type(16)));

constexpr int MX_WAVES = 8;
constexpr int MX_OPERAND = 64 * 16 + 64 * 8;        // bytes of one (half, q, term) operand: dwords 0-3, then dwords 4-5, per lane
constexpr int MX_SCALES = 8 * 3 * MX_OPERAND;       // the scale words of a Z buffer follow its 24 operands
constexpr int MX_ZBUF = MX_SCALES + 8 * 64 * 4;     // bytes per Z buffer

// raw buffer descriptor from a pointer: no stride, no range limit short of 4 GiB (every offset used with it is checked
// by construction: rows clamped to M, columns to the unit)
__device__ __forceinline__ __amdgpu_buffer_rsrc_t mx_rsrc(const void *p) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, -1, 0x00020000);
}

__device__ __forceinline__ uint32_t mx_and_or(uint32_t w, uint32_t mask, uint32_t base) { return (w & mask) | base; }

__device__ __forceinline__ float4_t mx_mfma(const uint4_t &a03, const uint2_t &a45, const uint4_t &b, float4_t c,
                                            int term, uint32_t scale_a, uint32_t scale_b) {
    const v8i_t av = {(int)a03[0], (int)a03[1], (int)a03[2], (int)a03[3], (int)a45[0], (int)a45[1], 0, 0};
    const v8i_t bv = {(int)b[0], (int)b[1], (int)b[2], (int)b[3], 0, 0, 0, 0};
    // A fp6 e2m3 (cbsz 2), B fp4 e2m1 (blgp 4); the A scale is byte `term` of scale_a
    switch (term) {
        case 0: return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(av, bv, c, 2, 4, 0, (int)scale_a, 0, (int)scale_b);
        case 1: return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(av, bv, c, 2, 4, 1, (int)scale_a, 0, (int)scale_b);
        default: return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(av, bv, c, 2, 4, 2, (int)scale_a, 0, (int)scale_b);
    }
}

// Production of the Z operands of one half unit (512 columns) for FOUR ranks by one wave: every vt
// value of a unit is loaded exactly once per workgroup, by coalesced 16-byte loads (load k is rank
// 4 j + k, lane l the 8 columns 8 l .. 8 l + 7 of the half unit; x likewise, one piece per lane).
// Of a piece's 8 products, position q uses columns 7 - q and 3 - q (negated for q = 3).  The pairs
// go through a transpose in a staging area private to the wave, so that lane (rank k', group g',
// position q') ends up with the 32 values z[2 b + hh], b = 0..15, of ONE MFMA operand lane; those
// are split into three fp6 terms and written where consumer lane 16 g' + rank reads them.
constexpr int MX_STAGE_BLK = 20;                     // dwords per staged (rank, position, group) block: 16 + 4, so that the
                                                     // 16-byte reads of 8 consecutive lanes hit 8 different bank groups
constexpr int MX_STAGE = 64 * MX_STAGE_BLK * 4;      // bytes of staging per wave
__device__ __forceinline__ void mx_produce_finish(char *zbuf, uint32_t *stage, const half8_t (&pv)[4], const half8_t &px,
                                                  int h, int j, int lane) {
    {
        const int g = lane >> 4, b = lane & 15;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            // (ranks beyond K carry a copy of rank K - 1: the flush multiplies them by u = 0)
            const half8_t p = pv[k] * px;
#pragma unroll
            for (int q = 0; q < 4; q++) {
                half2_t pr = {p[7 - q], p[3 - q]};
                if (q == 3) pr = -pr;
                stage[((k * 4 + q) * 4 + g) * MX_STAGE_BLK + b] = __builtin_bit_cast(uint32_t, pr);
            }
        }
    }
    // the reads below are of another type than the stores above: keep the compiler from moving them up
    // (the LDS operations of one wave execute in order, so no wait is needed)
    asm volatile("" ::: "memory");
    const int k = lane & 3, g = (lane >> 2) & 3, q = lane >> 4;
    uint4_t zw[4];
#pragma unroll
    for (int e = 0; e < 4; e++) zw[e] = *reinterpret_cast<const uint4_t *>(stage + ((k * 4 + q) * 4 + g) * MX_STAGE_BLK + 4 * e);
    // Block maximum of |z| on the BIT PATTERNS (unsigned 16-bit compare: monotonic for magnitudes, and
    // Inf = 0x7C00 < every NaN), so a NaN or an infinity in vt * x is seen instead of being dropped the way
    // a floating-point max drops NaN.  fp6 has no encoding for either: a block that holds one gets the
    // E8M0 scale 0xFF (NaN) on all three terms, every product of the block is NaN, and so is every output
    // that the column contributes to - as F.linear, and the fp16 kernel, give a non-finite result there.
    v16u_t zwords;
    ushort2_t mxb = {0, 0};
#pragma unroll
    for (int b = 0; b < 16; b++) {
        const uint32_t word = zw[b >> 2][b & 3];
        zwords[b] = word;
        mxb = __builtin_elementwise_max(mxb, __builtin_bit_cast(ushort2_t, word & 0x7FFF7FFFu));
    }
    const half32_t z = __builtin_bit_cast(half32_t, zwords);
    const uint16_t mbits = mxb[0] > mxb[1] ? mxb[0] : mxb[1];
    const bool finite = mbits < 0x7C00u;
    const float m = (float)__builtin_bit_cast(half_t, mbits);
    // exponent of s1 = floor(log2(m * 16 / 15)) - 2: the conversions use the exponent only
    const float s1 = finite ? fmaxf(m * (4.f / 15.f), 0x1p-100f) : 1.f, s2 = s1 * 0x1p-4f, s3 = s1 * 0x1p-8f;
    const uint32_t e1 = __builtin_bit_cast(uint32_t, s1) >> 23;
    const uint32_t scale = finite ? (e1 | ((e1 - 4u) << 8) | ((e1 - 8u) << 16)) : 0x00FFFFFFu;
    // residuals pair by pair (v_pk_add_f16): a subtraction of whole 32-element vectors is scalarised by the compiler
    auto minus = [](const half32_t &a, const half32_t &b) {
        const v16u_t aw = __builtin_bit_cast(v16u_t, a), bw = __builtin_bit_cast(v16u_t, b);
        v16u_t rw;
#pragma unroll
        for (int e = 0; e < 16; e++) {
            const uint32_t ae = aw[e], be = bw[e];
            rw[e] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, ae) - __builtin_bit_cast(half2_t, be));
        }
        return __builtin_bit_cast(half32_t, rw);
    };
    const v6u_t t1 = __builtin_amdgcn_cvt_scalef32_pk32_fp6_f16(z, s1);
    const half32_t r1 = minus(z, __builtin_amdgcn_cvt_scalef32_pk32_f16_fp6(t1, s1));
    const v6u_t t2 = __builtin_amdgcn_cvt_scalef32_pk32_fp6_f16(r1, s2);
    const half32_t r2 = minus(r1, __builtin_amdgcn_cvt_scalef32_pk32_f16_fp6(t2, s2));
    const v6u_t t3 = __builtin_amdgcn_cvt_scalef32_pk32_fp6_f16(r2, s3);
    const int hq = 4 * h + q, cl = 16 * g + 4 * j + k;             // operand set and consumer lane this thread feeds
    char *op = zbuf + hq * 3 * MX_OPERAND;
    *reinterpret_cast<uint4_t *>(op + cl * 16) = (uint4_t){t1[0], t1[1], t1[2], t1[3]};
    *reinterpret_cast<uint2_t *>(op + 1024 + cl * 8) = (uint2_t){t1[4], t1[5]};
    *reinterpret_cast<uint4_t *>(op + MX_OPERAND + cl * 16) = (uint4_t){t2[0], t2[1], t2[2], t2[3]};
    *reinterpret_cast<uint2_t *>(op + MX_OPERAND + 1024 + cl * 8) = (uint2_t){t2[4], t2[5]};
    *reinterpret_cast<uint4_t *>(op + 2 * MX_OPERAND + cl * 16) = (uint4_t){t3[0], t3[1], t3[2], t3[3]};
    *reinterpret_cast<uint2_t *>(op + 2 * MX_OPERAND + 1024 + cl * 8) = (uint2_t){t3[4], t3[5]};
    *reinterpret_cast<uint32_t *>(zbuf + MX_SCALES + hq * 256 + cl * 4) = scale;
}

// T = 1: a unit is 1024 columns of one token, its two 512-column halves produced by waves 0-3 and 4-7.
// T = 2: a unit is 512 columns of two tokens, token t produced by waves 4 t .. 4 t + 3; the eight
// operand sets of a Z buffer are then (token, position) instead of (half, position), everything else -
// LDS layout, passes, MFMA count per unit - is the same, and one set of sign words feeds both tokens.
template <int R, int T>
__global__ __launch_bounds__(64 * MX_WAVES, 1) void gemv_mx_kernel(
    const GemvGroup grp, const half_t *__restrict__ x, int N, int K, int n_units) {
    static_assert(T == 1 || T == 2, "one or two tokens");
    constexpr int UC = MX_UNIT_COLS / T;           // columns per unit
    constexpr int RW = MX_WAVES * R * 16;          // rows per workgroup
    constexpr int TG = R < 4 ? R : 4;              // row tiles whose sign operands are live together
    extern __shared__ __attribute__((aligned(16))) char lds[];
    char *zl = lds;                                                            // [2][MX_ZBUF]
    float *corrl = reinterpret_cast<float *>(lds + 2 * MX_ZBUF + MX_WAVES * MX_STAGE);   // [2][MX_WAVES][16]

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lm = lane & 15, g = lane >> 4;

    // XCD-aware slot -> range (workgroups are dealt round-robin to the 8 XCDs; each XCD gets a
    // contiguous run of ranges), then the matrix of the group this workgroup belongs to
    int wg;
    {
        const int nb = gridDim.x, xcd = blockIdx.x & 7, loc = blockIdx.x >> 3;
        const int base = nb >> 3, rem = nb & 7;
        wg = xcd * base + min(xcd, rem) + loc;
    }
    GemvMat mat = grp.m[0];
#pragma unroll
    for (int j = 1; j < GEMV_MAX_GROUP; j++)
        if (j < grp.n && wg >= grp.m[j].first_wg) mat = grp.m[j];
    wg -= mat.first_wg;
    const uint8_t *__restrict__ packed = mat.packed;
    const half_t *__restrict__ u = mat.u;
    const half_t *__restrict__ vt = mat.vt;
    float *__restrict__ part = mat.part;
    const int M = mat.M, row_tiles = mat.row_tiles, kmax = mat.kmax;
    const Split sp = mat.sp;
    const int u_begin = sp.start(wg), u_end = sp.start(wg + 1);
    if (u_begin >= u_end) return;

    const int64_t row_bytes = N >> 3;
    // producer role: half unit (T = 1) or token (T = 2) wave / 4, ranks 4 (wave % 4) .. + 3
    const int ph = wave >> 2, pj = wave & 3;
    uint32_t *stage = reinterpret_cast<uint32_t *>(lds + 2 * MX_ZBUF + wave * MX_STAGE);

    // a unit whose second half lies beyond N (N a multiple of 512 only) reads the first half's
    // addresses again there; x counts as zero for those columns, so they add nothing
    auto half_cols = [&](int c, int h) { return (T == 1 && c * UC + 512 * h < N) ? 512 * h : 0; };

    // ---- the unit being loaded: (block li, row tile, 1024-column chunk lc) ------------------------
    // Sign words and vt pieces are requested for the unit AFTER the one being multiplied; `qoff`,
    // `lq`, `lv` always describe that unit.
    uint32_t qoff[R];           // this lane's row in each row tile of the wave, as a byte offset within a block
    // Requests are raw buffer loads: a descriptor over the unit's origin (scalar registers), a 32-bit lane offset and a
    // scalar offset - no 64-bit address arithmetic in the vector unit, which this kernel cannot hide under its MFMAs.
    __amdgpu_buffer_rsrc_t lq;  // packed signs of the block, from the unit's first column
    __amdgpu_buffer_rsrc_t lv;  // vt of the block: rank 0, from the first column of half ph of the unit
    __amdgpu_buffer_rsrc_t lx;  // x (of token ph when T = 2) from the same column
    int l_h1;                   // byte offset of the unit's second half of a row (0 when it lies beyond N)
    bool l_xlive;               // the producer half of this wave lies within N
    auto set_unit = [&](int rowid, int c, bool new_row) {
        const int i = rowid / row_tiles;
        if (new_row) {
            const int rt = rowid - i * row_tiles;
#pragma unroll
            for (int jr = 0; jr < R; jr++) {
                const uint32_t row = (uint32_t)min(rt * RW + (wave * R + jr) * 16 + lm, M - 1);
                qoff[jr] = row * (uint32_t)row_bytes + 16u * g;
            }
        }
        lq = mx_rsrc(packed + (int64_t)i * M * row_bytes + c * (UC >> 3));
        l_h1 = half_cols(c, 1) >> 3;
        lv = mx_rsrc(vt + (int64_t)i * K * N + c * UC + half_cols(c, ph));
        lx = mx_rsrc(x + (T == 2 ? (int64_t)ph * N : 0) + c * UC + half_cols(c, ph));
        l_xlive = T == 2 || c * UC + 512 * ph < N;
    };

    float4_t acc[R][T];
    float4_t corr;              // this wave's operand set belongs to one token (T = 2: token wave / 4)
    auto clear_acc = [&]() {
        corr = (float4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int jr = 0; jr < R; jr++)
#pragma unroll
            for (int t = 0; t < T; t++) acc[jr][t] = (float4_t){0.f, 0.f, 0.f, 0.f};
    };
    clear_acc();

    half8_t pv[4], px;          // in flight: vt of rank 4 pj + k and x, columns 8 lane .. 8 lane + 7 of this wave's half unit
    auto produce_issue = [&](int c) {
        // (ranks beyond K repeat rank K - 1 and are zeroed when the operands are formed: no branch around a load)
#pragma unroll
        for (int k = 0; k < 4; k++)
            pv[k] = __builtin_bit_cast(half8_t, __builtin_amdgcn_raw_buffer_load_b128(lv, 16 * lane, min(4 * pj + k, K - 1) * N * 2, 0));
        px = __builtin_bit_cast(half8_t, __builtin_amdgcn_raw_buffer_load_b128(lx, 16 * lane, 0, 0));
    };
    auto produce_write = [&](int buf) {
        if (!l_xlive) px = (half8_t){0, 0, 0, 0, 0, 0, 0, 0};
        mx_produce_finish(zl + buf * MX_ZBUF, stage, pv, px, ph, pj, lane);
    };

    // ---- one (half, position) pass: per row tile four ANDs and three MFMAs ---------------------------
    // The sign words of a half unit are used by its four passes; in the last of them (q = 3, the
    // sign position, whose codes need the OR) every word is re-requested for the next unit right
    // behind its last use, so the sign bytes need one register set, not two.  (Unconditionally: a
    // branch around a load makes the compiler keep both values and wait for everything in flight.)
    // (w & 0x88888888) | 0x22222222 as ONE v_and_or_b32: VOP3 takes no literal and one scalar operand, so the mask is
    // pinned into a scalar register and the code of 1.0 into a vector register (empty asm statements the optimiser
    // cannot see through; the merge itself stays an ordinary expression the hazard recogniser can see)
    uint32_t sign_mask = 0x88888888u, ones_v = 0x22222222u;
    asm("" : "+s"(sign_mask));
    asm("" : "+v"(ones_v));
    uint4_t w[R][2];
    uint4_t bk[R];              // T = 2: the sign operands of a position, made for token 0 and used again for token 1
    auto pass = [&](const uint4_t &p0, const uint4_t &p1, const uint4_t &p2, const uint2_t &r0, const uint2_t &r1,
                    const uint2_t &r2, uint32_t sa, auto hq_const) {
        constexpr int h = decltype(hq_const)::value >> 2, q = decltype(hq_const)::value & 3;
        constexpr int wi = T == 1 ? h : 0, ti = T == 1 ? 0 : h;      // sign word set and token of this pass
        constexpr bool last_use = q == 3 && (T == 1 || h == 1);
        constexpr uint32_t mask = 0x11111111u << q;
        // B scale that makes a set bit worth 2 (q < 3: codes 2, 1, 0.5) or the sign code worth 1
        constexpr uint32_t sb = q == 3 ? 127u : 129u - q;
#pragma unroll
        for (int j0 = 0; j0 < R; j0 += TG) {
            uint4_t b[TG];
#pragma unroll
            for (int jr = 0; jr < TG; jr++) {
                if (T == 2 && h == 1) {
                    b[jr] = bk[j0 + jr];
                } else {
#pragma unroll
                    for (int p = 0; p < 4; p++) b[jr][p] = q == 3 ? mx_and_or(w[j0 + jr][wi][p], sign_mask, ones_v) : (w[j0 + jr][wi][p] & mask);
                    if (T == 2) bk[j0 + jr] = b[jr];
                }
                if (last_use) w[j0 + jr][wi] = __builtin_amdgcn_raw_buffer_load_b128(lq, (int)qoff[j0 + jr], wi ? l_h1 : 0, 0);
            }
            // term by term over the row tiles: consecutive MFMAs never share an accumulator
#pragma unroll
            for (int jr = 0; jr < TG; jr++) acc[j0 + jr][ti] = mx_mfma(p0, r0, b[jr], acc[j0 + jr][ti], 0, sa, sb);
#pragma unroll
            for (int jr = 0; jr < TG; jr++) acc[j0 + jr][ti] = mx_mfma(p1, r1, b[jr], acc[j0 + jr][ti], 1, sa, sb);
#pragma unroll
            for (int jr = 0; jr < TG; jr++) acc[j0 + jr][ti] = mx_mfma(p2, r2, b[jr], acc[j0 + jr][ti], 2, sa, sb);
            // pin the products to this pass: the optimiser otherwise sinks all MFMAs of a unit below the
            // operand reads of all its passes (the scheduling fences bind the instruction scheduler only)
#pragma unroll
            for (int jr = 0; jr < TG; jr++) asm volatile("" : "+v"(acc[j0 + jr][ti]));
        }
    };
    // The three fp6 terms of this lane's Z operand for a pass (dwords 0-3 and 4-5 of each) and their scale
    // word, in two register sets: operands are fetched one pass ahead.  Plain variables and explicit
    // passes: kept in a struct, or left to the unroller, they end up in scratch memory or all in
    // registers at once; the scheduling fences keep the eight passes apart.
#define MX_FETCH(S, HQ)                                                                                            \
    do {                                                                                                           \
        const char *op_ = zbuf + (HQ) * 3 * MX_OPERAND;                                                            \
        S##p0 = *reinterpret_cast<const uint4_t *>(op_ + lane * 16);                                               \
        S##r0 = *reinterpret_cast<const uint2_t *>(op_ + 1024 + lane * 8);                                         \
        S##p1 = *reinterpret_cast<const uint4_t *>(op_ + MX_OPERAND + lane * 16);                                  \
        S##r1 = *reinterpret_cast<const uint2_t *>(op_ + MX_OPERAND + 1024 + lane * 8);                            \
        S##p2 = *reinterpret_cast<const uint4_t *>(op_ + 2 * MX_OPERAND + lane * 16);                              \
        S##r2 = *reinterpret_cast<const uint2_t *>(op_ + 2 * MX_OPERAND + 1024 + lane * 8);                        \
        S##sa = *reinterpret_cast<const uint32_t *>(zbuf + MX_SCALES + (HQ) * 256 + lane * 4);                     \
    } while (0)
#define MX_PASS(S, HQ)                                                                                             \
    do {                                                                                                           \
        pass(S##p0, S##p1, S##p2, S##r0, S##r1, S##r2, S##sa, std::integral_constant<int, HQ>{});                   \
        __builtin_amdgcn_sched_barrier(0);                                                                         \
    } while (0)
    auto consume = [&](int buf) {
        const char *zbuf = zl + buf * MX_ZBUF;
        uint4_t fa_p0, fa_p1, fa_p2, fb_p0, fb_p1, fb_p2;
        uint2_t fa_r0, fa_r1, fa_r2, fb_r0, fb_r1, fb_r2;
        uint32_t fa_sa, fb_sa;
        // operand sets in the order they are multiplied: half by half (T = 1), or position by position with
        // both tokens of a position back to back (T = 2: set 4 t + q), so the sign operand is formed once
        constexpr int O1 = T == 1 ? 1 : 4, O2 = T == 1 ? 2 : 1, O3 = T == 1 ? 3 : 5, O4 = T == 1 ? 4 : 2,
                      O5 = T == 1 ? 5 : 6, O6 = T == 1 ? 6 : 3;
        MX_FETCH(fa_, 0);
        MX_FETCH(fb_, O1);
        MX_PASS(fa_, 0);
        MX_FETCH(fa_, O2);
        MX_PASS(fb_, O1);
        MX_FETCH(fb_, O3);
        MX_PASS(fa_, O2);
        MX_FETCH(fa_, O4);
        MX_PASS(fb_, O3);
        MX_FETCH(fb_, O5);
        MX_PASS(fa_, O4);
        MX_FETCH(fa_, O6);
        MX_PASS(fb_, O5);
        MX_FETCH(fb_, 7);
        MX_PASS(fa_, O6);
        MX_PASS(fb_, 7);
        // For the positions whose codes are 1 + s the accumulators also hold the sum of z over the
        // position's columns.  It does not depend on the row: wave w adds it up for operand set w
        // (one MFMA per term against the constant operand 1.0), the shares meet at flush time.
        if ((wave & 3) != 3) {
            constexpr uint32_t ONES = 0x22222222u;
            const uint4_t ones = {ONES, ONES, ONES, ONES};
            MX_FETCH(fa_, wave);
            corr = mx_mfma(fa_p0, fa_r0, ones, corr, 0, fa_sa, 127u);
            corr = mx_mfma(fa_p1, fa_r1, ones, corr, 1, fa_sa, 127u);
            corr = mx_mfma(fa_p2, fa_r2, ones, corr, 2, fa_sa, 127u);
        }
    };
#undef MX_FETCH
#undef MX_PASS

    // D[r, m]: the lane holds ranks 4g..4g+3 of row (tile jr, lm).  Subtract the correction
    // (summed over waves in a fixed order), scale by u, add the four lane groups, write the
    // partial row sum, start the next row from zero.
    // The u rows a flush multiplies by are requested one unit earlier (before the last unit of the row is
    // multiplied): requested inside the flush, every wave sat out their whole latency there.
    half4_t uc[R];
    auto request_u = [&](int rowid) {
        const int i = rowid / row_tiles, rt = rowid % row_tiles;
#pragma unroll
        for (int jr = 0; jr < R; jr++) {
            const int row = min(rt * RW + (wave * R + jr) * 16 + lm, M - 1);
            const half_t *up = u + ((int64_t)i * M + row) * K;
            if (K == 16) {
                uc[jr] = *reinterpret_cast<const half4_t *>(up + 4 * g);
            } else {
                // (ranks beyond K repeat rank K - 1 and are zeroed: no branch around a load)
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    const half_t val = up[min(4 * g + v, K - 1)];
                    uc[jr][v] = (4 * g + v < K) ? val : (half_t)0;
                }
            }
        }
    };
    int flush_parity = 0;
    auto flush = [&](int rowid, bool row_done) {
        // two flushes can follow each other with no barrier in between, so the exchange area alternates
        float *cx = corrl + flush_parity * (MX_WAVES * 16);
        flush_parity ^= 1;
        const int i = rowid / row_tiles, rt = rowid % row_tiles;
        if (lm == 0) *reinterpret_cast<float4_t *>(cx + wave * 16 + 4 * g) = corr;
        __syncthreads();
        const int slot = wg - sp.owner(rowid * n_units);
#pragma unroll
        for (int t = 0; t < T; t++) {
            // the corrections of this token: all eight waves' shares (T = 1), or those of waves 4 t .. 4 t + 3
            float4_t cz = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ww = 0; ww < MX_WAVES / T; ww++)
                cz += *reinterpret_cast<const float4_t *>(cx + (t * (MX_WAVES / T) + ww) * 16 + 4 * g);
#pragma unroll
            for (int jr = 0; jr < R; jr++) {
                const int row = rt * RW + (wave * R + jr) * 16 + lm;
                float val = (acc[jr][t][0] - cz[0]) * (float)uc[jr][0] + (acc[jr][t][1] - cz[1]) * (float)uc[jr][1] +
                            (acc[jr][t][2] - cz[2]) * (float)uc[jr][2] + (acc[jr][t][3] - cz[3]) * (float)uc[jr][3];
                val += __shfl_xor(val, 16, 64);
                val += __shfl_xor(val, 32, 64);
                if (g == 0 && row < M) {
                    part[(((int64_t)i * kmax + slot) * T + t) * M + row] = val;
                    // the workgroup that finishes a row of units zero-fills the slots above its own (nobody writes
                    // them): the summing kernel adds all kmax slots blindly
                    if (row_done)
                        for (int dead = slot + 1; dead < kmax; dead++) part[(((int64_t)i * kmax + dead) * T + t) * M + row] = 0.f;
                }
            }
        }
        clear_acc();
    };

    // ---- pipeline fill: first unit's signs and Z ----------------------------------------------
    int rowid = u_begin / n_units, c = u_begin % n_units;
    set_unit(rowid, c, true);
    produce_issue(c);
    // first halves first: the first four passes need nothing else (requests complete in order)
#pragma unroll
    for (int jr = 0; jr < R; jr++) w[jr][0] = __builtin_amdgcn_raw_buffer_load_b128(lq, (int)qoff[jr], 0, 0);
    if (T == 1) {
#pragma unroll
        for (int jr = 0; jr < R; jr++) w[jr][1] = __builtin_amdgcn_raw_buffer_load_b128(lq, (int)qoff[jr], l_h1, 0);
    }
    produce_write(0);
    __syncthreads();

    // ---- steady state ----------------------------------------------------------------------------
    int buf = 0;
    for (int unit = u_begin; unit + 1 < u_end; unit++) {
        const bool crossing = c + 1 == n_units;     // the next unit starts another row of units
        const int cn = crossing ? 0 : c + 1;
        if (crossing) request_u(rowid);             // the row ends with this unit
        set_unit(rowid + (crossing ? 1 : 0), cn, crossing);
        produce_issue(cn);
        __builtin_amdgcn_sched_barrier(0);
        consume(buf);
        produce_write(buf ^ 1);
        __syncthreads();
        if (crossing) {
            flush(rowid, true);
            rowid++;
        }
        c = cn;
        buf ^= 1;
    }
    // ---- drain ---------------------------------------------------------------------------------------
    request_u(rowid);
    __builtin_amdgcn_sched_barrier(0);
    consume(buf);          // (its refill requests repeat the last unit's addresses: valid, unused)
    flush(rowid, u_end % n_units == 0);
}

size_t mx_lds_bytes() { return (size_t)2 * MX_ZBUF + (size_t)MX_WAVES * MX_STAGE + 2 * MX_WAVES * 16 * sizeof(float); }

template <int R, int T>
int launch_mx(int grid, const GemvGroup &grp, const half_t *x, int N, int K, int n_units, hipStream_t s) {
    const size_t lds = mx_lds_bytes();
    static bs_lds_grant granted[BS_MAX_DEVICES];
    const int st = bs_allow_lds((const void *)gemv_mx_kernel<R, T>, lds, granted);
    if (st != BS_OK) return st;
    gemv_mx_kernel<R, T><<<grid, 64 * MX_WAVES, lds, s>>>(grp, x, N, K, n_units);
    BS_LAUNCH_CHECK();
    return BS_OK;
}

}  // namespace

// Shapes the block-scaled kernel runs: whole 512-column halves, one or two tokens.
bool bs_gemv_mx_takes(int N, int K, int R, int T) {
    if (N % 512 != 0 || K < 1 || K > 16 || T < 1 || T > 2) return false;
    return R == 1 || R == 2 || R == 4;
}

int bs_launch_gemv_mx(int R, int T, int grid, const GemvGroup &grp, const half_t *x, int N, int K, int n_units, hipStream_t s) {
    if (!bs_gemv_mx_takes(N, K, R, T) || n_units != (int)bs_cdiv(N, MX_UNIT_COLS / T)) return BS_ERR_SHAPE;
    if (T == 2) switch (R) {
        case 1: return launch_mx<1, 2>(grid, grp, x, N, K, n_units, s);
        case 2: return launch_mx<2, 2>(grid, grp, x, N, K, n_units, s);
        default: return launch_mx<4, 2>(grid, grp, x, N, K, n_units, s);
    }
    switch (R) {
        case 1: return launch_mx<1, 1>(grid, grp, x, N, K, n_units, s);
        case 2: return launch_mx<2, 1>(grid, grp, x, N, K, n_units, s);
        default: return launch_mx<4, 1>(grid, grp, x, N, K, n_units, s);
    }
}

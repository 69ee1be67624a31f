// Packed-sign GEMV for decode (1..8 tokens) on gfx950.
//
//   y[t, m] = sum_i sum_r u_i[m, r] * ( sum_n s_i[m, n] * vt_i[r, n] * x[t, n] )
//
// The inner sum is a matrix product  Z (16 ranks x N)  x  S^T (N x rows)  with
// Z[r, n] = vt_i[r, n] * x[t, n], so it runs on v_mfma_f32_16x16x32_f16:
// A = a 16 x 32 patch of Z (fp16), B = 32 signs of 16 rows, D[r, m] in fp32.
// A lane ends up with four ranks of ONE row, multiplies them by
// u_i[m, 4g..4g+3], and two cross-lane adds finish the row.
//
// ---- sign decode without shifts ------------------------------------------
// Decoding a bit to fp16 +-1 costs a shift and a mask per two signs, which is
// more VALU time than the MFMA it feeds.  Instead the bit is left WHERE IT IS
// in its 16-bit half and merged into a constant with one v_and_or_b32:
//     v = (w & (0x00010001 << j)) | base_j
// so the fp16 operand is one of two values {a_j, b_j} that depend on the bit
// position j, chosen such that b_j - a_j = 2 exactly:
//     j = 15 (sign)        {+1, -1}      mid  0   (Z is stored negated here)
//     j = 14 (exponent)    {0, 2}        mid  1
//     j = 9..4 (mantissa)  {4,6} {8,10} {16,18} {32,34} {64,66} {128,130}
// Then s = v - mid_j, and   sum_n s_n z_n = sum_n v_n z_n - sum_n mid_n z_n.
// The first sum is what the MFMAs accumulate; the second does not depend on
// the row; the waves of a workgroup share it out (16 / WAVES steps each, one extra
// MFMA per step against a constant operand) and exchange their shares through LDS
// when a row is flushed.  All codes are exact in fp16 and every product is exact
// in fp32, so the only extra error is fp32 accumulation of terms up to 129x
// larger than z (about 1e-5 relative, far below the fp16 rounding of y).
// Bit positions 10..13 and 0..3 have no such code (or a badly conditioned
// one), so the word is used three times: as loaded (positions 15,14,9..4),
// shifted left by 2 (positions 15,14 = original bits 13,12) and by 4
// (positions 15,14,7..4 = original bits 11,10,3..0): 2 shifts + 16 merges per
// 32 signs.
//
// ---- work split ------------------------------------------------------------
// The matrix stack is cut into UNITS: (block i, row tile of WAVES*R*16 rows,
// 512-column chunk), ordered with the chunk fastest.  The grid is persistent:
// about two workgroups per CU (one for three or four tokens), each owning one
// contiguous range of units of equal length, so the load is balanced for any
// shape and each workgroup pays its pipeline fill once.  Up to four matrices that
// read the same x share a launch: the grid is cut into one run of workgroups per
// matrix.  Per unit every lane reads its 16 bytes of signs
// (128 columns of one row) with one 128-bit load per row tile, one unit ahead
// of use; Z for unit u+1 is produced by all threads (vt and x loads issued
// before the MFMA loop of unit u, finished after it) into the other half of a
// double-buffered LDS image laid out in MFMA operand order: one barrier per
// unit.  Accumulators are flushed whenever the range crosses into another
// (block, row tile): scaled by u, reduced over ranks, written as a partial
// row sum to scratch [I, KMAX, T, M] (fp32); the workgroup that ends a row of
// units also writes zeros to the slots above its own (a row is spread over at
// most KMAX workgroups, often fewer).  A second kernel adds the KMAX slots of
// every block in a fixed order, adds the bias, rounds to fp16 and applies
// the epilogue (none, + residual, silu(a) * b): deterministic, no atomics.  Workgroups with neighbouring ranges - which read
// the same slices of vt - sit on the same XCD (and share its L2).
#include "common.h"
#include "gemv_shared.h"

#include <type_traits>
#include <utility>

namespace {

// Compile-time loop: the step tables below must fold to immediates.
template <class F, int... Is>
__device__ __forceinline__ void static_for_impl(F &&f, std::integer_sequence<int, Is...>) {
    (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F &&f) {
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}

constexpr int CH = 512;   // columns per chunk: 4 lane groups x 16 bytes of signs
constexpr int64_t MX_MIN_SIGN_BYTES = 8 << 20;   // sign bytes per launch from which the block-scaled kernel is preferred


// step -> bit position used in that step; steps 0-7 read the word as loaded,
// 8-9 after `<< 2`, 10-15 after `<< 4`.
__host__ __device__ constexpr int step_pos(int st) {
    constexpr int P[16] = {15, 14, 9, 8, 7, 6, 5, 4, 15, 14, 15, 14, 7, 6, 5, 4};
    return P[st];
}
// original bit (within its 16-bit half) -> step that consumes it
__host__ __device__ constexpr int bit_step(int b) {
    constexpr int S[16] = {15, 14, 13, 12, 7, 6, 5, 4, 3, 2, 11, 10, 9, 8, 1, 0};
    return S[b];
}
__host__ __device__ constexpr uint32_t pos_base(int j) {
    return j == 15 ? 0x3C003C00u : j == 14 ? 0u : j == 9 ? 0x44004400u : j == 8 ? 0x48004800u
         : j == 7 ? 0x4C004C00u : j == 6 ? 0x50005000u : j == 5 ? 0x54005400u : 0x58005800u;
}
__host__ __device__ constexpr float pos_mid(int j) {
    return j == 15 ? 0.f : j == 14 ? 1.f : j == 9 ? 5.f : j == 8 ? 9.f : j == 7 ? 17.f
         : j == 6 ? 33.f : j == 5 ? 65.f : 129.f;
}

// mid of the position each step reads (0 for the sign position)
__constant__ float step_mid_table[16] = {0.f, 1.f, 5.f, 9.f, 17.f, 33.f, 65.f, 129.f,
                                         0.f, 1.f, 0.f, 1.f, 17.f, 33.f, 65.f, 129.f};

// LDS image of Z for one chunk: [t][step (16)][g (4)][r (16)][slot (8)] halves.
__device__ inline int z_index(int t, int st, int g, int r) { return (((t * 16 + st) * 4 + g) * 16 + r) * 8; }

// (w & mask) | base as ONE v_and_or_b32.  VOP3 takes no literal and one scalar
// operand, so the two constants are first pinned into registers (mask scalar, base
// vector) with empty asm statements the optimiser cannot see through; the merge
// itself stays an ordinary expression.  It must not be written as an asm
// instruction: the compiler's hazard recogniser does not look inside inline asm,
// and a VALU write to registers that an MFMA issued just before still reads as its
// accumulator input (the MFMA reads SrcC several cycles after issue) corrupts that
// MFMA unless the recogniser can see the write and pad it.
__device__ inline uint32_t pin_scalar(uint32_t v) {
    asm("" : "+s"(v));
    return v;
}
__device__ inline uint32_t pin_vector(uint32_t v) {
    asm("" : "+v"(v));
    return v;
}
__device__ inline uint32_t and_or(uint32_t w, uint32_t mask, uint32_t base) { return (w & mask) | base; }

// One producer item: rank r, lane group pg, word p, byte pair (JB, JB + 2) of
// the word.  Two 16-byte pieces of vt (8 consecutive columns each) times x
// give 8 (slot 2p, slot 2p+1) pairs, one per bit of the byte.
template <int JB>
__device__ inline void produce_finish(half_t *zt, int pg, int p, int r, half8_t v0, half8_t v1,
                                      half8_t x0, half8_t x1) {
    const half8_t z0 = v0 * x0, z1 = v1 * x1;
    static_for<8>([&](auto ec) {
        constexpr int e = decltype(ec)::value;
        constexpr int st = bit_step(8 * JB + 7 - e);
        constexpr bool neg = step_pos(st) == 15;
        half2_t o = {z0[e], z1[e]};
        if (neg) o = -o;
        *reinterpret_cast<half2_t *>(zt + z_index(0, st, pg, r) + 2 * p) = o;
    });
}

template <int T, int WAVES, int R>
__global__ __launch_bounds__(64 * WAVES, (T == 1 ? (WAVES == 16 ? 1 : WAVES == 4 && R == 4 ? 3 : 4) : (T == 2 ? (WAVES == 8 && R == 2 ? 4 : 2) : 1))) void gemv_kernel(
    const GemvGroup grp, const half_t *__restrict__ x, int N, int K, int n_chunks) {
    constexpr int RW = WAVES * R * 16;          // rows per workgroup
    constexpr int COMBOS = WAVES >= 8 ? 1 : 8 / WAVES;   // (jb, pg) producer combos per wave (waves 8.. of 16 have none)
    constexpr int ZHALVES = T * 16 * 4 * 16 * 8;   // one Z buffer
    constexpr int CSTEPS = 16 / WAVES;          // correction steps handled by each wave
    extern __shared__ __attribute__((aligned(16))) half_t lds[];
    half_t *zl = lds;                                              // [2][ZHALVES]
    float *corrl = reinterpret_cast<float *>(lds + 2 * ZHALVES);   // [2][WAVES][T][16], alternating per flush

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform, keep it scalar
    const int lm = lane & 15, g = lane >> 4;

    // XCD-aware slot -> range: hardware deals workgroups round-robin to 8 XCDs;
    // give each XCD a contiguous run of ranges.
    int wg;
    {
        const int nb = gridDim.x, xcd = blockIdx.x & 7, loc = blockIdx.x >> 3;
        const int base = nb >> 3, rem = nb & 7;
        wg = xcd * base + min(xcd, rem) + loc;
    }
    // which matrix this workgroup belongs to (all of it is wave-uniform)
    GemvMat mat = grp.m[0];
#pragma unroll
    for (int j = 1; j < GEMV_MAX_GROUP; j++)
        if (j < grp.n && wg >= grp.m[j].first_wg) mat = grp.m[j];
    wg -= mat.first_wg;
    const int pair = mat.pair, cq = pair ? (wg & 1) : 0;      // chunk parity this workgroup takes
    const int wv = wg >> pair;                                // its place in the partition
    const int nch = n_chunks >> pair;                         // units per row of units
    const uint8_t *__restrict__ packed = mat.packed;
    const half_t *__restrict__ u = mat.u;
    const half_t *__restrict__ vt = mat.vt;
    float *__restrict__ part = mat.part;
    const int M = mat.M, row_tiles = mat.row_tiles, kmax = mat.kmax;
    const Split sp = mat.sp;
    const int u_begin = sp.start(wv), u_end = sp.start(wv + 1);
    if (u_begin >= u_end) return;

    const int64_t row_bytes = N >> 3;
    const int pp = lane & 3, pr = lane >> 2;      // producer role: word, rank
    const bool r_live = pr < K;

    // Addresses are a wave-uniform base (block i, kept in scalar registers) plus a
    // 32-bit per-lane byte offset that only changes with the row tile.
    const uint8_t *qbase;       // packed signs of block i
    const half_t *vbase;
    uint32_t qoff[R];           // this lane's row in each row tile of the wave
    const uint32_t voff = ((uint32_t)(r_live ? pr : 0) * (uint32_t)N + 32u * pp) * 2u;   // producer role
    auto set_row = [&](int rowid) {
        const int i = rowid / row_tiles, rt = rowid % row_tiles;
        qbase = packed + (int64_t)i * M * row_bytes;
        vbase = vt + (int64_t)i * K * N;
#pragma unroll
        for (int jr = 0; jr < R; jr++) {
            const uint32_t row = (uint32_t)min(rt * RW + (wave * R + jr) * 16 + lm, M - 1);
            qoff[jr] = row * (uint32_t)row_bytes + 16u * g;
        }
    };
    auto mid_operand = [&](int k) {   // constant MFMA operand for the correction sums of this wave's steps
        const half_t m = (half_t)step_mid_table[wave * CSTEPS + k];
        return (half8_t){m, m, m, m, m, m, m, m};
    };

    float4_t acc[R][T];
    float4_t corr[T];
    auto clear_acc = [&]() {
#pragma unroll
        for (int t = 0; t < T; t++) {
            corr[t] = (float4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int jr = 0; jr < R; jr++) acc[jr][t] = (float4_t){0.f, 0.f, 0.f, 0.f};
        }
    };
    clear_acc();

    half8_t pv[COMBOS][2];        // vt pieces in flight for the next unit
    half8_t px[COMBOS][T][2];     // x pieces in flight for the next unit
    auto produce_issue = [&](int c) {
        if (WAVES > 8 && wave >= 8) return;
#pragma unroll
        for (int k = 0; k < COMBOS; k++) {
            const int combo = wave + k * WAVES, pg = combo & 3, jb = combo >> 2;
            const int col = c * CH + 128 * pg + 8 * jb;            // wave-uniform
            const uint8_t *vs = reinterpret_cast<const uint8_t *>(vbase + col) + voff;
            pv[k][0] = *reinterpret_cast<const half8_t *>(vs);
            pv[k][1] = *reinterpret_cast<const half8_t *>(vs + 32);
#pragma unroll
            for (int t = 0; t < T; t++) {
                const uint8_t *xs = reinterpret_cast<const uint8_t *>(x + (int64_t)t * N + col) + 64u * pp;
                px[k][t][0] = *reinterpret_cast<const half8_t *>(xs);
                px[k][t][1] = *reinterpret_cast<const half8_t *>(xs + 32);
            }
        }
    };
    auto produce_write = [&](int buf) {
        if (WAVES > 8 && wave >= 8) return;
        half_t *zbuf = zl + buf * ZHALVES;
#pragma unroll
        for (int k = 0; k < COMBOS; k++) {
            const int combo = wave + k * WAVES, pg = combo & 3, jb = combo >> 2;
            half8_t v0 = pv[k][0], v1 = pv[k][1];
            if (!r_live) { v0 = (half8_t){0, 0, 0, 0, 0, 0, 0, 0}; v1 = v0; }
#pragma unroll
            for (int t = 0; t < T; t++) {
                half_t *zt = zbuf + z_index(t, 0, 0, 0);
                if (jb) produce_finish<1>(zt, pg, pp, pr, v0, v1, px[k][t][0], px[k][t][1]);
                else    produce_finish<0>(zt, pg, pp, pr, v0, v1, px[k][t][0], px[k][t][1]);
            }
        }
    };

    auto consume = [&](uint4_t (&w)[R], int buf) {
        const half_t *zbuf = zl + buf * ZHALVES;
        // Z fragments are fetched one step ahead of the MFMAs that use them: all
        // waves of a workgroup leave the barrier together, so nobody else would
        // cover the LDS latency.
        half8_t zf[2][T];
#pragma unroll
        for (int t = 0; t < T; t++) zf[0][t] = *reinterpret_cast<const half8_t *>(zbuf + z_index(t, 0, g, lm));
        static_for<16>([&](auto stc) {
            constexpr int st = decltype(stc)::value;
            if (st + 1 < 16) {
#pragma unroll
                for (int t = 0; t < T; t++)
                    zf[(st + 1) & 1][t] = *reinterpret_cast<const half8_t *>(zbuf + z_index(t, st + 1, g, lm));
            }
            if (st == 8 || st == 10) {
#pragma unroll
                for (int jr = 0; jr < R; jr++) w[jr] = w[jr] << 2;
            }
            constexpr int j = step_pos(st);
            constexpr uint32_t mask_c = 0x00010001u << j;
            const uint32_t mask = pin_scalar(mask_c), base = j == 14 ? 0u : pin_vector(pos_base(j));
#pragma unroll
            for (int jr = 0; jr < R; jr++) {
                uint4_t sb;
#pragma unroll
                for (int p = 0; p < 4; p++) sb[p] = (j == 14) ? (w[jr][p] & mask) : and_or(w[jr][p], mask, base);
                const half8_t sf = __builtin_bit_cast(half8_t, sb);
#pragma unroll
                for (int t = 0; t < T; t++)
                    acc[jr][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(zf[st & 1][t], sf, acc[jr][t], 0, 0, 0);
            }
        });
        // row-independent correction: this wave's share of the 16 steps
#pragma unroll
        for (int k = 0; k < CSTEPS; k++) {
#pragma unroll
            for (int t = 0; t < T; t++) {
                const half8_t zc = *reinterpret_cast<const half8_t *>(zbuf + z_index(t, wave * CSTEPS + k, g, lm));
                corr[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(zc, mid_operand(k), corr[t], 0, 0, 0);
            }
        }
    };

    auto load_signs = [&](uint4_t (&w)[R], int c) {
#pragma unroll
        for (int jr = 0; jr < R; jr++) w[jr] = *reinterpret_cast<const uint4_t *>(qbase + c * (CH >> 3) + qoff[jr]);
    };

    // D[r, m]: the lane holds ranks 4g..4g+3 of row (tile jr, lm).  Subtract the
    // correction (summed over waves in a fixed order), scale by u, add the four
    // lane groups, write the partial row sum, start the next row from zero.
    int flush_parity = 0;
    auto flush = [&](int rowid, bool row_done) {
        // Two flushes can follow each other with no barrier in between (a row that
        // ends on the last prefetching unit, then the drain), so the exchange area
        // alternates: a wave still reading the previous sums is never overwritten.
        float *cx = corrl + flush_parity * (WAVES * T * 16);
        flush_parity ^= 1;
        const int i = rowid / row_tiles, rt = rowid % row_tiles;
        half4_t uc[R];      // u[i, row, 4g .. 4g+3]
#pragma unroll
        for (int jr = 0; jr < R; jr++) {
            const int row = min(rt * RW + (wave * R + jr) * 16 + lm, M - 1);
            const half_t *up = u + ((int64_t)i * M + row) * K + 4 * g;
            if (K == 16) {
                uc[jr] = *reinterpret_cast<const half4_t *>(up);
            } else {
#pragma unroll
                for (int v = 0; v < 4; v++) uc[jr][v] = (4 * g + v < K) ? up[v] : (half_t)0;
            }
        }
        if (lm == 0) {
#pragma unroll
            for (int t = 0; t < T; t++) *reinterpret_cast<float4_t *>(cx + (wave * T + t) * 16 + 4 * g) = corr[t];
        }
        __syncthreads();
        const int slot = ((wv - sp.owner(rowid * nch)) << pair) + cq;
#pragma unroll
        for (int t = 0; t < T; t++) {
            float4_t cz = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int w = 0; w < WAVES; w++) cz += *reinterpret_cast<const float4_t *>(cx + (w * T + t) * 16 + 4 * g);
#pragma unroll
            for (int jr = 0; jr < R; jr++) {
                const int row = rt * RW + (wave * R + jr) * 16 + lm;
                float val = (acc[jr][t][0] - cz[0]) * (float)uc[jr][0] + (acc[jr][t][1] - cz[1]) * (float)uc[jr][1] +
                            (acc[jr][t][2] - cz[2]) * (float)uc[jr][2] + (acc[jr][t][3] - cz[3]) * (float)uc[jr][3];
                val += __shfl_xor(val, 16, 64);
                val += __shfl_xor(val, 32, 64);
                if (g == 0 && row < M) {
                    part[(((int64_t)i * kmax + slot) * T + t) * M + row] = val;
                    // The workgroup that finishes a row of units holds its highest live slot: it fills the
                    // slots nobody writes with zeros, so the summing kernel adds all kmax slots blindly.
                    if (row_done)
                        for (int dead = slot + (1 << pair); dead < kmax; dead += 1 << pair)
                            part[(((int64_t)i * kmax + dead) * T + t) * M + row] = 0.f;
                }
            }
        }
        clear_acc();
    };

    // ---- pipeline fill: first unit's signs and Z -----------------------------
    int rowid = u_begin / nch, c = u_begin % nch;
    set_row(rowid);
    uint4_t cur[R], nxt[R];
    auto chunk_of = [&](int unit_c) { return (unit_c << pair) + cq; };   // unit within its row -> 512-column chunk
    produce_issue(chunk_of(c));                     // first: Z production only waits for these
    load_signs(cur, chunk_of(c));
    uint32_t warm0;      // loaded for its side effect only (the line ends up in L2)
    {
        // the flush after the last unit is not preceded by a crossing inside the loop:
        // pull the u rows it needs towards L2 now (value unused)
        const int lrow = (u_end - 1) / nch, fi = lrow / row_tiles, frt = lrow % row_tiles;
        const int frow = min(frt * RW + wave * (R * 16) + (lane & (R * 16 - 1)), M - 1);
        warm0 = *reinterpret_cast<const uint32_t *>(u + ((int64_t)fi * M + frow) * K);
    }
    produce_write(0);
    __syncthreads();
    asm volatile("" ::"v"(warm0));                  // keeps the load; by now it has long arrived

    // ---- steady state -------------------------------------------------------
    int buf = 0;
    uint32_t warm_in = 0;
    for (int unit = u_begin; unit + 1 < u_end; unit++) {
        const bool crossing = c + 1 == nch;         // the next unit starts another row
        const int cn = crossing ? 0 : c + 1;
        if (crossing) {
            // the row ends with this unit: pull its u rows towards L2 now (one
            // dword per row, value unused) so the flush below does not wait on HBM
            const int fi = rowid / row_tiles, frt = rowid % row_tiles;
            const int frow = min(frt * RW + wave * (R * 16) + (lane & (R * 16 - 1)), M - 1);
            warm_in = *reinterpret_cast<const uint32_t *>(u + ((int64_t)fi * M + frow) * K);
            set_row(rowid + 1);                     // address arithmetic only
        }
        produce_issue(chunk_of(cn));                // L2-resident: first, so waiting for them does not wait for HBM
        load_signs(nxt, chunk_of(cn));
        __builtin_amdgcn_sched_barrier(0);          // keep the prefetch at the top of the unit
        consume(cur, buf);
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("" ::"v"(warm_in));              // keeps the load alive; waited for only here, behind the MFMA loop
        produce_write(buf ^ 1);
        __syncthreads();
        if (crossing) {
            flush(rowid, true);
            rowid++;
        }
#pragma unroll
        for (int jr = 0; jr < R; jr++) cur[jr] = nxt[jr];
        c = cn;
        buf ^= 1;
    }
    // ---- drain: last unit, nothing left to prefetch -----------------------------
    consume(cur, buf);
    flush(rowid, u_end % nch == 0);
}

// y[t, off + m] = epilogue( fp16( sum_i sum_k part[i, k, t, m] + bias[m] ) ): every one of the I * kmax
// slots of an output holds a number (the decode kernels zero-fill the slots nobody needed; the strip
// kernels write one partial per strip group, I = groups and kmax = 1), added up in a fixed order.
// Epilogues (applied to the fp16-rounded sums, the way separate fp16 ops would):
//   EPI_NONE      the matrices' outputs side by side in one row of `ldy` halves
//   EPI_RESIDUAL  the same plus residual[t, off + m]
//   EPI_SWIGLU    two matrices of equal M: silu(first) * second, one row of M
constexpr int RED_MAXBLOCKS = 1024;      // a sanity limit on the block count

struct RedMat {
    const float *part;
    const half_t *bias;
    int I, M, kmax, y_off, first_block;
};
struct RedGroup {
    RedMat m[GEMV_MAX_GROUP];
    int n, mode;
    // input RMS scale: when xin is set, every sum is multiplied by rsqrt(mean(xin[t, :]^2) + eps)
    // before the bias - the scalar half of an RMSNorm in front of the matrices (its weight
    // vector belongs folded into vt by the caller)
    const half_t *xin;
    int n_in;
    float eps;
    // the same scale from ready-made partial sums of squares, ssq[g * T + t] for g < ssq_n
    // (written by the strip kernel); takes precedence over xin
    const float *ssq;
    int ssq_n;
};

// No slot counts, no divisions, and the loads of a thread depend on nothing but its index, so the
// kernel is one memory round trip long.  A workgroup produces 256 / SL consecutive outputs of one
// token; SL threads per output take every SL-th of the I * kmax slots (SL = 1: no LDS, no barrier).
// SCALED: the input RMS scale of RedGroup::xin or RedGroup::ssq.
constexpr int FLAT_BATCH = 8;
template <int SL>
__device__ __forceinline__ float flat_slice_sum(const RedMat &r, int T, int t, int m, int ks) {
    const int total = r.I * r.kmax;
    const int64_t stride = (int64_t)T * r.M;
    const float *base = r.part + (int64_t)t * r.M + m;
    float acc = 0.f;
    for (int s0 = ks; s0 < total; s0 += FLAT_BATCH * SL) {
        float v[FLAT_BATCH];
#pragma unroll
        for (int j = 0; j < FLAT_BATCH; j++) {
            const int s = s0 + j * SL;
            v[j] = base[(int64_t)(s < total ? s : 0) * stride];
        }
#pragma unroll
        for (int j = 0; j < FLAT_BATCH; j++) acc += (s0 + j * SL < total) ? v[j] : 0.f;
    }
    return acc;
}

template <int SL, bool SCALED>
__global__ __launch_bounds__(256) void gemv_reduce_flat_kernel(
    const RedGroup grp, const half_t *__restrict__ residual, half_t *__restrict__ y, int T, int ldy) {
    constexpr int RUN = 256 / SL;
    __shared__ float red[2][SL][RUN];
    __shared__ float ssq[4];
    const int lo = threadIdx.x % RUN, ks = threadIdx.x / RUN;
    const bool two = grp.mode == EPI_SWIGLU;
    int j = 0;
    if (!two) {
#pragma unroll
        for (int q = 1; q < GEMV_MAX_GROUP; q++)
            if (q < grp.n && (int)blockIdx.x >= grp.m[q].first_block) j = q;
    }
    const RedMat &r = grp.m[j];
    const int local = blockIdx.x - r.first_block;
    const int per_t = (r.M + RUN - 1) / RUN;
    const int t = local / per_t, m = (local - t * per_t) * RUN + lo;
    const bool live = m < r.M;
    // everything this thread reads is requested before anything is waited for
    float s0 = live ? flat_slice_sum<SL>(r, T, t, m, ks) : 0.f;
    float s1 = (two && live) ? flat_slice_sum<SL>(grp.m[1], T, t, m, ks) : 0.f;
    float extra0 = 0.f, extra1 = 0.f, res = 0.f;
    if (ks == 0 && live) {
        if (r.bias) extra0 = (float)r.bias[m];
        if (two && grp.m[1].bias) extra1 = (float)grp.m[1].bias[m];
        if (grp.mode == EPI_RESIDUAL) res = (float)residual[(int64_t)t * ldy + r.y_off + m];
    }
    float scale = 1.f;
    if (SCALED) {
        float q = 0.f;
        if (grp.ssq) {                           // sums of squares per strip group, left by the strip kernel
            for (int c = threadIdx.x; c < grp.ssq_n; c += 256) q += grp.ssq[c * T + t];
        } else {
            const half_t *xr = grp.xin + (int64_t)t * grp.n_in;
            for (int c = threadIdx.x * 8; c < grp.n_in; c += 256 * 8) {
                const half8_t v = *reinterpret_cast<const half8_t *>(xr + c);
#pragma unroll
                for (int e = 0; e < 8; e++) q += (float)v[e] * (float)v[e];
            }
        }
#pragma unroll
        for (int o = 32; o >= 1; o >>= 1) q += __shfl_xor(q, o, 64);
        if ((threadIdx.x & 63) == 0) ssq[threadIdx.x >> 6] = q;
    }
    if (SL > 1) {
        red[0][ks][lo] = s0;
        if (two) red[1][ks][lo] = s1;
    }
    if (SL > 1 || SCALED) __syncthreads();
    if (SCALED) scale = rsqrtf((ssq[0] + ssq[1] + ssq[2] + ssq[3]) / (float)grp.n_in + grp.eps);
    if (ks != 0 || !live) return;
    if (SL > 1) {
        s0 = 0.f;
        s1 = 0.f;
#pragma unroll
        for (int k = 0; k < SL; k++) s0 += red[0][k][lo];
        if (two) {
#pragma unroll
            for (int k = 0; k < SL; k++) s1 += red[1][k][lo];
        }
    }
    const float a0 = s0 * scale + extra0;
    if (two) {
        const float a1 = s1 * scale + extra1;
        const float gate = (float)(half_t)a0, up = (float)(half_t)a1;
        const half_t act = (half_t)(gate / (1.f + __expf(-gate)));
        y[(int64_t)t * ldy + m] = (half_t)((float)act * up);
    } else {
        half_t v = (half_t)a0;
        if (grp.mode == EPI_RESIDUAL) v = (half_t)(res + (float)v);
        y[(int64_t)t * ldy + r.y_off + m] = v;
    }
}

template <int SL>
void launch_reduce_flat(int blocks, const RedGroup &r, const half_t *residual, half_t *y, int T, int ldy, hipStream_t s) {
    if (r.xin || r.ssq)
        gemv_reduce_flat_kernel<SL, true><<<blocks, 256, 0, s>>>(r, residual, y, T, ldy);
    else
        gemv_reduce_flat_kernel<SL, false><<<blocks, 256, 0, s>>>(r, residual, y, T, ldy);
}

struct Plan {
    int waves, R, n_chunks, grid, n, pair;
    int mx;        // 1: the block-scaled fp4 x fp6 kernel (gemv_mx.hip), units of MX_UNIT_COLS columns
    int row_tiles[GEMV_MAX_GROUP], kmax[GEMV_MAX_GROUP], first_wg[GEMV_MAX_GROUP];
    Split sp[GEMV_MAX_GROUP];
    int64_t part_off[GEMV_MAX_GROUP];      // in floats; part_off[n] = total
    int64_t part_total;
};

// One instantiation and one grid for the whole group; every matrix gets a share of
// the workgroups in proportion to its units.
// Which kernel make_plan picks for one and two tokens: 0 by shape, 1 always the fp16 kernel, 2 the block-scaled one
// wherever it takes the shape (bs_set_decode_kernel, for tests and benchmarks).  Per calling thread: a size query
// and the forward behind it on one thread agree whatever other threads set.
thread_local int g_decode_kernel = 0;

// Rows per workgroup of the block-scaled kernel for these matrices (0: it does not run them).
int mx_rows_per_tile(const int *I, const int *M, int n, int N, int K, int T) {
    if (g_decode_kernel == 1 || !bs_gemv_mx_takes(N, K, 1, T)) return 0;
    const int n_units = (int)bs_cdiv(N, MX_UNIT_COLS / T);
    int pick = 0;
    for (int r = 4; r >= 1; r >>= 1) {
        const int rw = 8 * r * 16;
        bool tall = true;
        int64_t units = 0;
        for (int j = 0; j < n; j++) {
            tall = tall && M[j] >= rw;
            units += bs_cdiv(M[j], rw) * I[j] * n_units;
        }
        if ((tall && units >= 256) || r == 1) { pick = r; break; }
    }
    if (g_decode_kernel == 2) return pick;
    // by shape: the long-stack cases, where the contraction loop and not the fixed cost of a launch decides
    int64_t bytes = 0;
    for (int j = 0; j < n; j++) bytes += (int64_t)I[j] * M[j] * (N / 8);
    return (pick >= 2 && bytes >= MX_MIN_SIGN_BYTES) ? pick : 0;
}

Plan make_plan(const int *I, const int *M, int n, int N, int K, int T) {
    Plan p;
    p.n = n;
    p.n_chunks = N / CH;
    p.mx = 0;
    const int mx_r = mx_rows_per_tile(I, M, n, N, K, T);
    if (mx_r > 0) {
        // one workgroup of 8 waves per CU; units are (block, row tile, 1024 columns), never paired
        p.mx = 1;
        p.waves = 8;
        p.R = mx_r;
        p.pair = 0;
        p.n_chunks = (int)bs_cdiv(N, MX_UNIT_COLS / T);
        int units[GEMV_MAX_GROUP], total = 0, biggest = 0;
        for (int j = 0; j < n; j++) {
            p.row_tiles[j] = (int)bs_cdiv(M[j], 8 * mx_r * 16);
            units[j] = I[j] * p.row_tiles[j] * p.n_chunks;
            total += units[j];
            if (units[j] > units[biggest]) biggest = j;
        }
        int grid = total < 256 ? total : 256, gj[GEMV_MAX_GROUP], sum = 0;
        for (int j = 0; j < n; j++) {
            gj[j] = n == 1 ? grid : (int)(((int64_t)grid * units[j] + total / 2) / total);
            if (gj[j] < 1) gj[j] = 1;
            if (gj[j] > units[j]) gj[j] = units[j];
            sum += gj[j];
        }
        while (sum > grid && gj[biggest] > 1) { gj[biggest]--; sum--; }
        int first = 0;
        int64_t off = 0;
        for (int j = 0; j < n; j++) {
            p.first_wg[j] = first;
            first += gj[j];
            p.sp[j].q = units[j] / gj[j];
            p.sp[j].rem = units[j] % gj[j];
            int kmax = (int)bs_cdiv(p.n_chunks - 1, p.sp[j].q) + 1;
            if (kmax > gj[j]) kmax = gj[j];
            p.kmax[j] = kmax;
            p.part_off[j] = off;
            off += (int64_t)I[j] * kmax * T * M[j];
        }
        p.grid = first;
        p.part_total = off;
        return p;
    }
    // rows per workgroup: 512 (8 waves x 4 tiles), 256, 128, 64; resident workgroups per CU.
    // Three or four tokens need more than the 128 registers a lane has with two 8-wave
    // workgroups per CU: there it is one workgroup of 8 waves per CU (two waves per SIMD
    // to overlap sign decode and MFMA), four row tiles per wave (each Z fragment read
    // from LDS feeds four MFMAs per token) or two when the layer has too few units.
    const int cand1[4][3] = {{8, 4, 2}, {4, 4, 3}, {4, 2, 4}, {4, 1, 4}};
    const int wide1[3] = {16, 4, 1};
    const int cand3[4][3] = {{8, 4, 1}, {8, 2, 1}, {4, 2, 1}, {4, 1, 1}};
    const int cand2[4][3] = {{8, 2, 2}, {4, 4, 2}, {4, 2, 2}, {4, 1, 2}};
    const int (*cand)[3] = T > 2 ? cand3 : T == 2 ? cand2 : cand1;
    int pick = 3;
    for (int k = 0; k < 4; k++) {
        const int rw = cand[k][0] * cand[k][1] * 16;
        bool tall = true;
        int64_t units = 0;
        for (int j = 0; j < n; j++) {
            tall = tall && M[j] >= rw;
            units += bs_cdiv(M[j], rw) * I[j] * p.n_chunks;
        }
        // enough units that every CU gets one
        if (tall && units >= 256) { pick = k; break; }
    }
    // One token, long stacks: one workgroup of 16 waves per CU.  Two 8-wave workgroups on a CU do
    // not share it evenly (the older one is served first and finishes a third earlier, the
    // younger one then runs on a half-empty CU); sixteen waves that meet at one barrier do.
    const int *choice = cand[pick];
    if (T == 1) {
        bool tall = true;
        int64_t units = 0;
        for (int j = 0; j < n; j++) {
            tall = tall && M[j] >= 1024;
            units += bs_cdiv(M[j], 1024) * I[j] * p.n_chunks;
        }
        if (tall && units >= GEMV_WIDE_MIN_UNITS) choice = wide1;
    }
    p.waves = choice[0];
    p.R = choice[1];
    int units[GEMV_MAX_GROUP], total = 0;
    for (int j = 0; j < n; j++) {
        p.row_tiles[j] = (int)bs_cdiv(M[j], p.waves * p.R * 16);
        units[j] = I[j] * p.row_tiles[j] * p.n_chunks;
        total += units[j];
    }
    int grid = 256 * (T == 1 ? choice[2] : T == 2 ? 2 : 1);
    // prefer two units per workgroup (one pipeline fill amortised over two units) as
    // long as every CU still gets a workgroup
    if (grid > total / 2) grid = total / 2 >= 256 ? total / 2 : (total < 256 ? total : 256);
    if (grid < 1) grid = 1;
    // Paired workgroups (GemvMat::pair) once a workgroup has several units to stream: the
    // grid is then a multiple of 16, so that the contiguous run of workgroups an XCD gets
    // starts and ends on a pair.
    p.pair = (p.n_chunks % 2 == 0 && total >= GEMV_PAIR_MIN_UNITS * grid && grid >= 16 * n) ? 1 : 0;
    int gj[GEMV_MAX_GROUP], sum = 0, biggest = 0;
    for (int j = 0; j < n; j++) {
        gj[j] = n == 1 ? grid : (int)(((int64_t)grid * units[j] + total / 2) / total);
        if (p.pair) gj[j] &= ~1;
        if (gj[j] < 1 + p.pair) gj[j] = 1 + p.pair;
        if (gj[j] > units[j]) gj[j] = units[j];
        sum += gj[j];
        if (units[j] > units[biggest]) biggest = j;
    }
    if (p.pair) {
        // round the grid to a multiple of 16 on the largest matrix (down when it can spare them)
        const int over = sum % 16;
        if (over && gj[biggest] > over + 16) gj[biggest] -= over;
        else if (over && gj[biggest] + 16 - over <= units[biggest]) gj[biggest] += 16 - over;
        else if (over) p.pair = 0;
        if (!p.pair)      // back to the plain plan
            for (int j = 0; j < n; j++) {
                gj[j] = n == 1 ? grid : (int)(((int64_t)grid * units[j] + total / 2) / total);
                if (gj[j] < 1) gj[j] = 1;
                if (gj[j] > units[j]) gj[j] = units[j];
            }
    }
    if (!p.pair && n > 1) {
        // rounding per matrix may leave one workgroup too many: it would wait for a free slot
        // and run after the others (a launch of 513 takes a fifth longer than one of 512)
        sum = 0;
        for (int j = 0; j < n; j++) sum += gj[j];
        while (sum > grid && gj[biggest] > 1) { gj[biggest]--; sum--; }
    }
    int first = 0;
    int64_t off = 0;
    for (int j = 0; j < n; j++) {
        const int places = gj[j] >> p.pair, uj = units[j] >> p.pair, nch = p.n_chunks >> p.pair;
        p.first_wg[j] = first;
        first += gj[j];
        p.sp[j].q = uj / places;
        p.sp[j].rem = uj % places;
        // most places a row of nch units can be spread over
        int kmax = (int)bs_cdiv(nch - 1, p.sp[j].q) + 1;
        if (kmax > places) kmax = places;
        p.kmax[j] = kmax << p.pair;
        p.part_off[j] = off;
        off += (int64_t)I[j] * p.kmax[j] * T * M[j];
    }
    p.grid = first;
    p.part_total = off;
    return p;
}

struct GroupArgs {          // host-side view of one call
    int n;
    const uint8_t *packed[GEMV_MAX_GROUP];
    const half_t *u[GEMV_MAX_GROUP], *vt[GEMV_MAX_GROUP], *bias[GEMV_MAX_GROUP];
    int I[GEMV_MAX_GROUP], M[GEMV_MAX_GROUP];
};

template <int T, int WAVES, int R>
int launch_one(const Plan &p, const GemvGroup &grp, const half_t *x, int N, int K, hipStream_t s) {
    const size_t lds = (size_t)2 * T * 16384 + (size_t)2 * WAVES * T * 64;
    static bs_lds_grant granted[BS_MAX_DEVICES];      // per instantiation
    const int st = bs_allow_lds((const void *)gemv_kernel<T, WAVES, R>, lds, granted);
    if (st != BS_OK) return st;
    gemv_kernel<T, WAVES, R><<<p.grid, 64 * WAVES, lds, s>>>(grp, x, N, K, p.n_chunks);
    BS_LAUNCH_CHECK();
    return BS_OK;
}

// Only the (WAVES, R) pairs make_plan can choose for T tokens exist; any other pair is refused
// rather than run on a tile of another height (the reduce kernel and the partial layout are
// built for exactly waves * R * 16 rows per tile).
template <int T>
int launch_T(const Plan &p, const GemvGroup &grp, const half_t *x, int N, int K, hipStream_t s) {
    const int w = p.waves, r = p.R;
    if constexpr (T == 1) {
        if (w == 16 && r == 4) return launch_one<1, 16, 4>(p, grp, x, N, K, s);
        if (w == 8 && r == 4) return launch_one<1, 8, 4>(p, grp, x, N, K, s);
    } else if constexpr (T == 2) {
        if (w == 8 && r == 2) return launch_one<2, 8, 2>(p, grp, x, N, K, s);
    } else {
        if (w == 8 && r == 4) return launch_one<T, 8, 4>(p, grp, x, N, K, s);
        if (w == 8 && r == 2) return launch_one<T, 8, 2>(p, grp, x, N, K, s);
    }
    if constexpr (T <= 2) {
        if (w == 4 && r == 4) return launch_one<T, 4, 4>(p, grp, x, N, K, s);
    }
    if (w == 4 && r == 2) return launch_one<T, 4, 2>(p, grp, x, N, K, s);
    if (w == 4 && r == 1) return launch_one<T, 4, 1>(p, grp, x, N, K, s);
    return BS_ERR_SHAPE;
}

bool gemv_shape_ok(int I, int M, int N, int T) {
    // per-block byte offsets are kept in 32 bits inside the kernel
    return I >= 1 && I <= RED_MAXBLOCKS && T >= 1 && T <= 8 && N % CH == 0 && M >= 1 &&
           (int64_t)M * N < ((int64_t)1 << 31);
}

// Tokens are processed in passes of at most four (LDS holds Z for four tokens).
int pass_tokens(int T) { return T <= 4 ? T : (T + 1) / 2; }

// From this many tokens on the strip kernel (weight patches rebuilt in registers and
// multiplied at once) is faster than passes of the factor-through kernel, which needs 16
// rank-MFMAs per token and patch where the strip kernel needs one for 16 tokens.
constexpr int STRIP_MIN_T = 5, STRIP_MAX_T = BS_PANEL_MAX_T;       // (49 tokens and more: the walked and panel kernels, single matrices only)

bool strip_group_ok(const int *I, const int *M, int n, int N, int K, int T) {
    for (int j = 0; j < n; j++)
        if (bs_strip_partials(I[j], M[j], N, K, T) == 0) return false;
    return true;
}
bool gemv_group_ok(const int *I, const int *M, int n, int N, int T) {
    for (int j = 0; j < n; j++)
        if (!gemv_shape_ok(I[j], M[j], N, T)) return false;
    return true;
}
// 1: strip kernel, 0: factor-through kernel, -1: neither takes the shapes
int group_path(const int *I, const int *M, int n, int N, int K, int T) {
    if (n < 1 || n > GEMV_MAX_GROUP) return -1;
    if (T >= STRIP_MIN_T && T <= STRIP_MAX_T && strip_group_ok(I, M, n, N, K, T)) return 1;
    if (gemv_group_ok(I, M, n, N, T)) return 0;
    return -1;
}
int64_t strip_part_floats(const int *I, const int *M, int n, int N, int K, int T) {
    int64_t total = (int64_t)bs_strip_partials(I[0], M[0], N, K, T) * T;      // sums of squares of x per strip group
    for (int j = 0; j < n; j++) total += (int64_t)bs_strip_partials(I[j], M[j], N, K, T) * T * M[j];
    return total;
}

// Strip path: one launch writes part[strip group, t, m] of every matrix; the reduce kernel
// reads that as "one partial per block" with the strip groups in the place of the blocks.
int launch_group_strips(const GroupArgs &a, int N, int K, const half_t *x, int T, int mode, const half_t *residual,
                        half_t *y, bool input_rms, float eps, void *workspace, int64_t workspace_bytes, hipStream_t s) {
    if (!workspace || workspace_bytes < strip_part_floats(a.I, a.M, a.n, N, K, T) * (int64_t)sizeof(float)) return BS_ERR_WORKSPACE;
    float *part = (float *)workspace;
    RedGroup r;
    r.n = a.n;
    r.mode = mode;
    r.xin = nullptr;
    r.n_in = N;
    r.eps = eps;
    float *parts[GEMV_MAX_GROUP];
    // threads per output of the summing kernel, as behind the decode kernels (the strip groups are its slots)
    int slots = 0;
    for (int j = 0; j < a.n; j++) {
        const int groups = bs_strip_partials(a.I[j], a.M[j], N, K, T);
        if (groups > slots) slots = groups;
    }
    const int sl = slots <= FLAT_BATCH ? 1 : slots <= 2 * FLAT_BATCH ? 2 : slots <= 4 * FLAT_BATCH ? 4 : 8;
    const int run = 256 / sl;
    int ldy = 0, blocks = 0;
    int64_t off = 0;
    for (int j = 0; j < a.n; j++) {
        const int groups = bs_strip_partials(a.I[j], a.M[j], N, K, T);
        parts[j] = part + off;
        r.m[j] = RedMat{part + off, a.bias[j], groups, a.M[j], 1, ldy, blocks};
        off += (int64_t)groups * T * a.M[j];
        ldy += a.M[j];
        if (mode != EPI_SWIGLU || j == 0) blocks += T * (int)bs_cdiv(a.M[j], run);
    }
    r.ssq = input_rms ? part + off : nullptr;
    r.ssq_n = r.m[0].I;
    const int st = bs_launch_strip_group(a.n, a.packed, a.u, a.vt, a.I, a.M, parts, input_rms ? part + off : nullptr,
                                         x, N, K, T, s);
    if (st != BS_OK) return st;
    if (mode == EPI_SWIGLU) ldy = a.M[0];
    for (int j = a.n; j < GEMV_MAX_GROUP; j++) r.m[j] = r.m[0];
    switch (sl) {
        case 1: launch_reduce_flat<1>(blocks, r, residual, y, T, ldy, s); break;
        case 2: launch_reduce_flat<2>(blocks, r, residual, y, T, ldy, s); break;
        case 4: launch_reduce_flat<4>(blocks, r, residual, y, T, ldy, s); break;
        default: launch_reduce_flat<8>(blocks, r, residual, y, T, ldy, s); break;
    }
    BS_LAUNCH_CHECK();
    return BS_OK;
}

int launch_group(const GroupArgs &a, int N, int K, const half_t *x, int T, int mode, const half_t *residual,
                 half_t *y, bool input_rms, float eps, void *workspace, int64_t workspace_bytes, hipStream_t s) {
    if (a.n < 1 || a.n > GEMV_MAX_GROUP) return BS_ERR_SHAPE;
    if (!bs_aligned(x, 16)) return BS_ERR_SHAPE;
    if (mode == EPI_SWIGLU && (a.n != 2 || a.M[0] != a.M[1])) return BS_ERR_SHAPE;
    const int path = group_path(a.I, a.M, a.n, N, K, T);
    if (path < 0) return BS_ERR_SHAPE;
    if (path == 1) {
        for (int j = 0; j < a.n; j++)
            if (!bs_aligned(a.packed[j], 16) || !bs_aligned(a.vt[j], 16) || !bs_aligned(a.u[j], 8)) return BS_ERR_SHAPE;
        return launch_group_strips(a, N, K, x, T, mode, residual, y, input_rms, eps, workspace, workspace_bytes, s);
    }
    int ldy = 0;
    for (int j = 0; j < a.n; j++) {
        if (!gemv_shape_ok(a.I[j], a.M[j], N, T)) return BS_ERR_SHAPE;
        if (!bs_aligned(a.packed[j], 16) || !bs_aligned(a.vt[j], 16) || !bs_aligned(a.u[j], 8)) return BS_ERR_SHAPE;
        ldy += a.M[j];
    }
    if (mode == EPI_SWIGLU) {
        if (a.n != 2 || a.M[0] != a.M[1]) return BS_ERR_SHAPE;
        ldy = a.M[0];
    }
    // Tokens go in passes of tp, the last one possibly shorter.  Every pass length has its own
    // plan (instantiation, grid, partial layout): the kernel a plan names exists for that token
    // count only.  Passes run one after the other on the stream and share the workspace.
    const int tp = pass_tokens(T);
    float *part = (float *)workspace;
    for (int t0 = 0; t0 < T; t0 += tp) {
        const int tn = (T - t0 < tp) ? T - t0 : tp;
        const Plan p = make_plan(a.I, a.M, a.n, N, K, tn);
        if (!workspace || workspace_bytes < p.part_total * (int64_t)sizeof(float)) return BS_ERR_WORKSPACE;
        GemvGroup g;
        RedGroup r;
        g.n = r.n = a.n;
        r.mode = mode;
        r.n_in = N;
        r.eps = eps;
        r.ssq = nullptr;
        r.ssq_n = 0;
        // threads per output of the summing kernel: at most FLAT_BATCH loads in flight per thread where the slots allow
        int slots = 0;
        for (int j = 0; j < a.n; j++)
            if (a.I[j] * p.kmax[j] > slots) slots = a.I[j] * p.kmax[j];
        const int sl = slots <= FLAT_BATCH ? 1 : slots <= 2 * FLAT_BATCH ? 2 : slots <= 4 * FLAT_BATCH ? 4 : 8;
        const int run = 256 / sl;
        int y_off = 0, blocks = 0;
        for (int j = 0; j < a.n; j++) {
            g.m[j] = GemvMat{a.packed[j], a.u[j], a.vt[j], part + p.part_off[j], a.M[j], p.row_tiles[j], p.kmax[j],
                             p.first_wg[j], p.sp[j], p.pair};
            r.m[j] = RedMat{part + p.part_off[j], a.bias[j], a.I[j], a.M[j], p.kmax[j], y_off, blocks};
            y_off += a.M[j];
            if (mode != EPI_SWIGLU || j == 0) blocks += tn * (int)bs_cdiv(a.M[j], run);
        }
        for (int j = a.n; j < GEMV_MAX_GROUP; j++) { g.m[j] = g.m[0]; r.m[j] = r.m[0]; }
        const half_t *xp = x + (int64_t)t0 * N;
        r.xin = input_rms ? xp : nullptr;
        int st;
        if (p.mx) st = bs_launch_gemv_mx(p.R, tn, p.grid, g, xp, N, K, p.n_chunks, s);
        else switch (tn) {
            case 1: st = launch_T<1>(p, g, xp, N, K, s); break;
            case 2: st = launch_T<2>(p, g, xp, N, K, s); break;
            case 3: st = launch_T<3>(p, g, xp, N, K, s); break;
            default: st = launch_T<4>(p, g, xp, N, K, s); break;
        }
        if (st != BS_OK) return st;
        const half_t *res_p = residual ? residual + (int64_t)t0 * ldy : nullptr;
        half_t *y_p = y + (int64_t)t0 * ldy;
        switch (sl) {
            case 1: launch_reduce_flat<1>(blocks, r, res_p, y_p, tn, ldy, s); break;
            case 2: launch_reduce_flat<2>(blocks, r, res_p, y_p, tn, ldy, s); break;
            case 4: launch_reduce_flat<4>(blocks, r, res_p, y_p, tn, ldy, s); break;
            default: launch_reduce_flat<8>(blocks, r, res_p, y_p, tn, ldy, s); break;
        }
        BS_LAUNCH_CHECK();
    }
    return BS_OK;
}

// Scratch the factor-through path needs: the largest partial area over its passes.
int64_t gemv_part_floats(const int *I, const int *M, int n, int N, int K, int T) {
    const int tp = pass_tokens(T), tail = T % tp;
    int64_t need = make_plan(I, M, n, N, K, tp).part_total;
    if (tail) {
        const int64_t t2 = make_plan(I, M, n, N, K, tail).part_total;
        if (t2 > need) need = t2;
    }
    return need;
}

}  // namespace

int64_t bs_gemv_workspace_bytes(int I, int M, int N, int K, int T) {
    return bs_gemv_group_workspace_bytes(&I, &M, 1, N, K, T);
}

// Bytes of scratch the packed-sign paths (factor-through or strip kernel) need for these
// matrices and token count; 0 when neither takes them.
int64_t bs_gemv_group_workspace_bytes(const int *I, const int *M, int n, int N, int K, int T) {
    const int path = group_path(I, M, n, N, K, T);
    if (path < 0) return 0;
    if (path == 1) return strip_part_floats(I, M, n, N, K, T) * (int64_t)sizeof(float);
    return gemv_part_floats(I, M, n, N, K, T) * (int64_t)sizeof(float);
}

// Which instantiation and grid a decode forward of these dimensions runs
// (0 in *waves when the decode kernel does not take them).
void bs_gemv_plan_info(int I, int M, int N, int K, int T, int *waves, int *row_tiles_per_wave, int *grid, int *kmax) {
    *waves = *row_tiles_per_wave = *grid = *kmax = 0;
    if (group_path(&I, &M, 1, N, K, T) != 0) return;
    const Plan p = make_plan(&I, &M, 1, N, K, pass_tokens(T));
    *waves = p.waves;
    *row_tiles_per_wave = p.R;
    *grid = p.grid;
    *kmax = p.kmax[0];
}

// The kernel family a single-matrix forward of these dimensions runs on (values of BS_PATH_* in the public header).
int bs_gemv_forward_path(int I, int M, int N, int K, int T) {
    const int path = group_path(&I, &M, 1, N, K, T);
    if (path < 0) return BS_PATH_REBUILD;
    if (path == 1) {
        const int c = bs_strip_kernel_choice(I, M, N, K, T);
        return c == 1 ? BS_PATH_STRIP : c == 2 ? BS_PATH_WALKED : BS_PATH_PANEL;
    }
    return make_plan(&I, &M, 1, N, K, pass_tokens(T)).mx ? BS_PATH_DECODE_MX : BS_PATH_DECODE_F16;
}

// 0: not a decode-kernel shape, 1: gemv_kernel (fp16 MFMA), 2: gemv_mx_kernel (block-scaled fp4 x fp6 MFMA)
int bs_gemv_plan_kernel(int I, int M, int N, int K, int T) {
    if (group_path(&I, &M, 1, N, K, T) != 0) return 0;
    return make_plan(&I, &M, 1, N, K, pass_tokens(T)).mx ? 2 : 1;
}

int bs_gemv_set_kernel(int mode) {
    if (mode < 0 || mode > 2) return BS_ERR_SHAPE;
    g_decode_kernel = mode;
    return BS_OK;
}

// Returns BS_ERR_SHAPE when the fast path does not apply (the caller falls
// back to rebuilding the weight); any other status is final.
int bs_launch_gemv(const uint8_t *packed, const half_t *u, const half_t *vt, const half_t *x,
                   const half_t *bias, half_t *y, int I, int M, int N, int K, int T,
                   void *workspace, int64_t workspace_bytes, hipStream_t s) {
    GroupArgs a;
    a.n = 1;
    a.packed[0] = packed; a.u[0] = u; a.vt[0] = vt; a.bias[0] = bias; a.I[0] = I; a.M[0] = M;
    return launch_group(a, N, K, x, T, EPI_NONE, nullptr, y, false, 0.f, workspace, workspace_bytes, s);
}

int bs_launch_gemv_group(int n, const uint8_t *const *packed, const half_t *const *u, const half_t *const *vt,
                         const half_t *const *bias, const int *I, const int *M, int N, int K, const half_t *x, int T,
                         int mode, const half_t *residual, half_t *y, int input_rms, float eps, void *workspace,
                         int64_t workspace_bytes, hipStream_t s) {
    if (n < 1 || n > GEMV_MAX_GROUP) return BS_ERR_SHAPE;
    if (mode == EPI_RESIDUAL && !residual) return BS_ERR_NULL;
    GroupArgs a;
    a.n = n;
    for (int j = 0; j < n; j++) {
        a.packed[j] = packed[j]; a.u[j] = u[j]; a.vt[j] = vt[j]; a.bias[j] = bias ? bias[j] : nullptr;
        a.I[j] = I[j]; a.M[j] = M[j];
    }
    return launch_group(a, N, K, x, T, mode, residual, y, input_rms != 0, eps, workspace, workspace_bytes, s);
}

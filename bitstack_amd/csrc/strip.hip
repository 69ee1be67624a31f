// Forward for a handful to a few dozen tokens on gfx950: the weight is rebuilt patch by
// patch in registers and multiplied by x at once; it never goes to memory.
//
//   part[strip, t, m] = sum_{n in strip} x[t, n] * fp16( sum_i s_i[m, n] * sum_r u_i[m, r] * vt_i[r, n] )
//
// Same decomposition as the weight rebuild (a workgroup owns a strip of 128 columns and
// a range of rows, the strip's slice of vt of ALL blocks staged transposed in LDS, per
// block one v_mfma_f32_16x16x16_f16 per 16 x 16 patch computed transposed, the signs of a
// nibble looked up as four halves of +-1.0 and multiplied in by a mixed-precision FMA).
// When the last block of a 16-row step is in, a lane
// holds w[m0 + lm, 4 consecutive columns] of each patch - exactly the B operand of a
// second v_mfma_f32_16x16x16_f16 whose A operand is x[16 tokens, the same 4 columns]
// (read from an LDS copy of the strip's slice of x) and whose result is y[token, row]
// for this strip.  w is rounded to fp16 before that product, as it is when it is stored
// and multiplied by the dense kernel.  The strips' partial sums go to scratch
// [strip, T, M] (fp32); the reduce kernel of the decode path adds them in strip order
// and applies bias and epilogue.
//
// Cost per 16 x 16 patch and block: the same 6 to 7 VALU operations as the rebuild, no store
// of w (two thirds of the rebuild's bytes) and no second pass that reads it back; the
// token count only adds one MFMA per patch and 16 tokens, after the last block.
#include "common.h"
#include "rebuild_shared.h"

namespace {

// Extra halves per token row of the x image: rows then start two banks apart, so the 16 tokens a quarter wave reads
// (8 bytes each, the same columns) fall on 32 different banks.  (With 8, tokens t and t + 8 shared their banks.)
// Rows are 8-byte aligned only: the image is written and read in pieces of four halves.
constexpr int XPAD = 4;

// TT = token tiles of 16.  A workgroup takes `sg` (1, 2, 4 or 8) neighbouring strips at once:
// their vt slices are staged together, and per 16-row step the partial y of all of them
// is added up in registers, so scratch holds one partial per GROUP of strips and a lane
// reads sg * 16 consecutive sign bytes of its row.
// Up to four matrices that read the same x share a launch (q/k/v, gate/up): the grid is cut
// into one run of slots per matrix, each with its own strips per workgroup and row split.
constexpr int STRIP_MAX_GROUP = 4;
struct StripMat {
    const uint8_t *packed;
    const half_t *u, *vt;
    float *part;
    int I, M, sg, rows_per_wg, row_groups, first_slot;
};
struct StripGroup {
    StripMat m[STRIP_MAX_GROUP];
    int n;
    float *ssq;     // [strip groups of matrix 0][T]: sum of x^2 over the group's columns (for an RMS scale), or null
};

// K16: the rank is 16 (every u fragment is one 8-byte load).  Smaller ranks pick their halves one by one behind
// branches, and the compiler then waits for every load in flight where the branches meet.
template <int TT, int WAVES, bool K16>
__global__ __launch_bounds__(64 * WAVES, 4) void strip_forward_kernel(
    const StripGroup grp, const half_t *__restrict__ x, int N, int K, int T) {
    extern __shared__ __attribute__((aligned(128))) half_t lds_all[];
    half_t *const lds = lds_all + SIGN_LUT_HALVES;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // the same in every lane: loop counts that depend on it stay scalar
    const int lm = lane & 15, g = lane >> 4;
    // Workgroups are dealt round-robin to the 8 XCDs.  Every matrix owns a run of block
    // indices that starts at a multiple of 8, so each XCD gets an eighth of every matrix
    // (their slots differ in work).  Within a matrix the slot order is (128-byte line of
    // sign bytes, row group, strip group within the line) in contiguous runs per XCD: the
    // 8 / sg groups that share a line meet in one L2.  Strip groups are padded to whole
    // lines and the slots to a multiple of 8; slots beyond the last strip idle.
    StripMat mat = grp.m[0];
    bool first_matrix = true;
    int slots = grp.n > 1 ? grp.m[1].first_slot : (int)gridDim.x;
#pragma unroll
    for (int j = 1; j < STRIP_MAX_GROUP; j++)
        if (j < grp.n && (int)blockIdx.x >= grp.m[j].first_slot) {
            mat = grp.m[j];
            first_matrix = false;
            slots = (j + 1 < grp.n ? grp.m[j + 1].first_slot : (int)gridDim.x) - mat.first_slot;
        }
    const int local = (int)blockIdx.x - mat.first_slot;
    const int slot = (local & 7) * (slots >> 3) + (local >> 3);
    const uint8_t *__restrict__ packed = mat.packed;
    const half_t *__restrict__ u = mat.u;
    const half_t *__restrict__ vt = mat.vt;
    float *__restrict__ part = mat.part;
    const int I = mat.I, M = mat.M, sg = mat.sg, rows_per_wg = mat.rows_per_wg;
    const int xstride = sg * SF_COLS + XPAD;        // halves per token row of the x image
    half_t *xl = lds;                               // [TT * 16][xstride]
    half_t *vl = lds + TT * 16 * xstride;           // [sg][I][VBLOCK]
    int group, row_begin;
    {
        const int per_line = 8 / sg, rest = slot / per_line;
        group = (rest / mat.row_groups) * per_line + slot % per_line;
        row_begin = (rest % mat.row_groups) * rows_per_wg;
    }
    const int strips = N / SF_COLS;
    const int s_begin = group * sg;
    if (s_begin >= strips) return;
    const int ns = min(sg, strips - s_begin);       // strips this workgroup really has
    const int n0 = s_begin * SF_COLS;
    const int row_end = min(row_begin + rows_per_wg, M);
    const int64_t row_bytes = N >> 3;
    const int64_t block_bytes = (int64_t)M * row_bytes;

    const int sr = tid & 15, sp = (tid >> 4) & 15;  // staging role: rank, piece of 8 columns
    const int spair = tid >> 8;                     // ... and which of the WAVES / 4 pairs staged side by side
    const SignTable st = make_sign_table(lds_all, tid, g);
    const int acol = 8 * (lm >> 2) + (lm & 3);
    const int aoff = acol * VSTRIDE + (lm >> 2) * VGROUP_PAD + 4 * g;

    const int first_row = row_begin + wave * 16;
    constexpr int NT = 64 * WAVES, RS = 16 * WAVES;  // threads, rows per step of the workgroup
    const int last_m0 = first_row + ((max(row_end - first_row, 1) - 1) / RS) * RS;
    // Addresses are a wave-uniform 64-bit base (block, strip: scalar arithmetic) plus a 32-bit
    // offset per lane that depends on the row only and is renewed once per row step; worked out
    // per request in 64 bits per lane, the multiplications were a fifth of the kernel's VALU time.
    uint32_t off_u, off_s;                          // bytes: this lane's u row (its four ranks) and sign row
    auto set_row = [&](int m0) {
        const int row = min(min(m0, last_m0) + lm, M - 1);
        off_u = (uint32_t)(row * K + 4 * g) * 2u;
        off_s = (uint32_t)row * (uint32_t)row_bytes;
    };
    auto load_block = [&](int i, int q, half4_t &b, uint4_t &sw) {
        const char *ub = reinterpret_cast<const char *>(u) + (int64_t)i * M * K * 2;
        const half_t *up = reinterpret_cast<const half_t *>(ub + off_u);
        if (K16) {
            b = *reinterpret_cast<const half4_t *>(up);
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++) b[j] = (4 * g + j < K) ? up[j] : (half_t)0;
        }
        const uint8_t *sb = packed + i * block_bytes + ((n0 + q * SF_COLS) >> 3);
        sw = *reinterpret_cast<const uint4_t *>(sb + off_s);
    };
    // The (row step, strip, block) triples of this wave form one sequence; its sign and u loads run
    // NS - 1 triples ahead, and they are unconditional (behind the last triple they repeat its row
    // step): a branch around a load makes the compiler wait for every load in flight at the join,
    // which left the waves waiting for data half of their time.
    // (three token tiles leave registers for two sets only)
    constexpr int NS = TT >= 3 ? 2 : NSETS;
    // One token tile at rank 16 has the registers for both code versions of a block: the first block of a strip starts
    // the sums (rebuild_block<true>) instead of adding to accumulators cleared behind the second product.
    constexpr bool PEEL = TT == 1 && K16;
    half4_t b_set[NS];
    uint4_t sw_set[NS];
#pragma unroll
    for (int k = 0; k < NS; k++) sw_set[k] = (uint4_t){0, 0, 0, 0};
    int pf_i = 0, pf_q = 0, pf_m0 = first_row;      // the triple the next request is for
    set_row(pf_m0);
    auto request = [&](half4_t &b, uint4_t &sw) {
        load_block(pf_i, pf_q, b, sw);
        if (++pf_i == I) {
            pf_i = 0;
            if (++pf_q == ns) {
                pf_q = 0;
                pf_m0 += RS;
                set_row(pf_m0);
            }
        }
    };
#pragma unroll
    for (int k = 0; k + 1 < NS; k++) request(b_set[k], sw_set[k]);

    // x image: token rows beyond T are zero
    for (int idx = tid; idx < TT * 16 * ns * 16; idx += NT) {
        const int t = idx / (ns * 16), piece = idx % (ns * 16);
        half8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
        if (t < T) v = *reinterpret_cast<const half8_t *>(x + (int64_t)t * N + n0 + 8 * piece);
        *reinterpret_cast<half4_t *>(xl + t * xstride + 8 * piece) = (half4_t){v[0], v[1], v[2], v[3]};
        *reinterpret_cast<half4_t *>(xl + t * xstride + 8 * piece + 4) = (half4_t){v[4], v[5], v[6], v[7]};
    }
    // vt slices, four (strip, block) pairs at a time so that their loads are in flight together
    constexpr int SIDE = WAVES / 4;                 // 256 threads stage one (strip, block) pair
    for (int q0 = 0; q0 < ns * I; q0 += 4 * SIDE) {
        half8_t v[4];
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const int qi = min(q0 + k * SIDE + spair, ns * I - 1), q = qi / I, i = qi - q * I;
            v[k] = (half8_t){0, 0, 0, 0, 0, 0, 0, 0};
            if (sr < K) v[k] = *reinterpret_cast<const half8_t *>(vt + ((int64_t)i * K + sr) * N + n0 + q * SF_COLS + 8 * sp);
        }
#pragma unroll
        for (int k = 0; k < 4; k++) {
            if (q0 + k * SIDE + spair < ns * I) {
#pragma unroll
                for (int e = 0; e < 8; e++) vl[(q0 + k * SIDE + spair) * VBLOCK + (8 * sp + e) * VSTRIDE + sp * VGROUP_PAD + sr] = v[k][e];
            }
        }
    }
    __syncthreads();

    // sum of squares of every token over this group's columns, once per strip group
    if (grp.ssq && first_matrix && row_begin == 0) {
        const int sub = tid & 7;
        // eight lanes per token row, NT / 8 rows per pass (48 token rows need two passes of 256 threads)
        for (int t0 = 0; t0 < TT * 16; t0 += NT / 8) {
            const int t = t0 + (tid >> 3);
            float q = 0.f;
            if (t < TT * 16) {
                for (int c = sub * 8; c < ns * SF_COLS; c += 64) {
                    const half4_t v0 = *reinterpret_cast<const half4_t *>(xl + t * xstride + c);
                    const half4_t v1 = *reinterpret_cast<const half4_t *>(xl + t * xstride + c + 4);
#pragma unroll
                    for (int e = 0; e < 4; e++) q += (float)v0[e] * (float)v0[e];
#pragma unroll
                    for (int e = 0; e < 4; e++) q += (float)v1[e] * (float)v1[e];
                }
            }
            q += __shfl_xor(q, 1, 64);
            q += __shfl_xor(q, 2, 64);
            q += __shfl_xor(q, 4, 64);
            if (sub == 0 && t < T) grp.ssq[group * T + t] = q;
        }
    }

    // this lane's x fragments: token lm of a tile, columns 32 (s / 2) + 8 g + 4 (s % 2) .. + 3 of patch s
    const half_t *xfrag = xl + lm * xstride + 8 * g;

    // the triple being consumed: rows m0.., strip q of the group, block i
    float4_t yacc[TT], acc[8];
#pragma unroll
    for (int tt = 0; tt < TT; tt++) yacc[tt] = (float4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < 8; s++) acc[s] = (float4_t){0.f, 0.f, 0.f, 0.f};
    int i = 0, q = 0, m0 = first_row;
    auto consume = [&](const half4_t &b, const uint4_t &sw) {
        const half_t *vb = vl + (q * I + i) * VBLOCK + aoff;
        if (PEEL && i == 0)
            rebuild_block<true>(vb, b, sw, st, acc);
        else
            rebuild_block<false>(vb, b, sw, st, acc);
        if (++i < I) return;
        i = 0;
        // y[token, row] of this strip: D[token 4g + v, row lm] = sum_k x[token, col(k)] * w[row, col(k)]
        const half_t *xq = xfrag + q * SF_COLS;
#pragma unroll
        for (int s = 0; s < 8; s++) {
            const half4_t wf = {(half_t)acc[s][0], (half_t)acc[s][1], (half_t)acc[s][2], (half_t)acc[s][3]};
            if (!PEEL) acc[s] = (float4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int tt = 0; tt < TT; tt++) {
                const half4_t xf = *reinterpret_cast<const half4_t *>(xq + tt * 16 * xstride + 32 * (s >> 1) + 4 * (s & 1));
                yacc[tt] = __builtin_amdgcn_mfma_f32_16x16x16f16(xf, wf, yacc[tt], 0, 0, 0);
            }
        }
        if (++q < ns) return;
        q = 0;
        if (m0 + lm < M) {
#pragma unroll
            for (int tt = 0; tt < TT; tt++)
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    const int t = 16 * tt + 4 * g + v;
                    if (t < T) part[((int64_t)group * T + t) * M + m0 + lm] = yacc[tt][v];
                }
        }
#pragma unroll
        for (int tt = 0; tt < TT; tt++) yacc[tt] = (float4_t){0.f, 0.f, 0.f, 0.f};
        m0 += RS;
    };
    const int n_triples = first_row < row_end ? ((row_end - first_row + RS - 1) / RS) * ns * I : 0;
    for (int p = 0; p < n_triples; p += NS) {
#pragma unroll
        for (int k = 0; k < NS; k++) {
            if (k > 0 && p + k >= n_triples) break;
            request(b_set[(k + NS - 1) % NS], sw_set[(k + NS - 1) % NS]);   // the set consumed last
            consume(b_set[k], sw_set[k]);
        }
    }
}

// ---- 49 to 96 tokens: the same patches, the strips walked by the workgroup -----------------------
// With more token tiles the partial sums of strip_forward_kernel ([strip group, T, M] floats) outgrow the
// weight itself, so here a workgroup keeps y[T, its 128 rows] in registers (TT accumulators per wave) and
// walks a run of strips: per chunk of `sg` strips it stages the x and vt slices in LDS (one barrier before,
// one after), every wave rebuilds its 16 rows of those strips patch by patch and multiplies them into the
// accumulators at once.  The weight never exists outside registers, and scratch holds one partial per
// COLUMN GROUP (a handful), not per strip.  The columns are cut into as many groups as it takes to fill the
// chip with workgroups of 128 rows; workgroups of one column group sit on one XCD and share its vt slices.
struct WideMat {
    const uint8_t *packed;
    const half_t *u, *vt;
    float *part;
    int I, M, sg, n_chunk, row_tiles;
};

template <int TT, bool K16>
__global__ __launch_bounds__(512, 4) void strip_wide_kernel(const WideMat mat, const half_t *__restrict__ x, int N, int K, int T) {
    constexpr int WAVES = 8, NT = 64 * WAVES, RS = 16 * WAVES;
    constexpr bool PEEL = false;                    // (no registers left for the two code versions of a block)
    extern __shared__ __attribute__((aligned(128))) half_t lds_all[];
    half_t *const lds = lds_all + SIGN_LUT_HALVES;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lm = lane & 15, g = lane >> 4;
    int cgroup, rt;
    {
        const int nb = gridDim.x, xcd = blockIdx.x & 7, loc = blockIdx.x >> 3;
        const int base = nb >> 3, rem = nb & 7;
        const int v = xcd * base + min(xcd, rem) + loc;
        cgroup = v / mat.row_tiles;
        rt = v - cgroup * mat.row_tiles;
    }
    const uint8_t *__restrict__ packed = mat.packed;
    const half_t *__restrict__ u = mat.u;
    const half_t *__restrict__ vt = mat.vt;
    const int I = mat.I, M = mat.M, sg = mat.sg, n_chunk = mat.n_chunk;
    const int xstride = sg * SF_COLS + XPAD;        // halves per token row of the x image
    half_t *xl = lds;                               // [TT * 16][xstride]
    half_t *vl = lds + TT * 16 * xstride;           // [sg][I][VBLOCK]
    const int strips = N / SF_COLS;
    const int first_strip = cgroup * n_chunk * sg;  // this workgroup's strips: first_strip .. + n_chunk * sg - 1, those below `strips`
    const int64_t row_bytes = N >> 3;
    const int64_t block_bytes = (int64_t)M * row_bytes;

    const int sr = tid & 15, sp = (tid >> 4) & 15;  // staging role: rank, piece of 8 columns
    const int spair = tid >> 8;                     // ... and which of the two (strip, block) pairs staged side by side
    const SignTable st = make_sign_table(lds_all, tid, g);
    const int acol = 8 * (lm >> 2) + (lm & 3);
    const int aoff = acol * VSTRIDE + (lm >> 2) * VGROUP_PAD + 4 * g;

    const int m0 = rt * RS + wave * 16;
    const int row = min(m0 + lm, M - 1);
    const uint32_t off_u = (uint32_t)(row * K + 4 * g) * 2u;              // bytes: this lane's u row (its four ranks) and sign row
    const uint32_t off_s = (uint32_t)row * (uint32_t)row_bytes;
    auto load_block = [&](int i, int strip, half4_t &b, uint4_t &sw) {
        const char *ub = reinterpret_cast<const char *>(u) + (int64_t)i * M * K * 2;
        const half_t *up = reinterpret_cast<const half_t *>(ub + off_u);
        if (K16) {
            b = *reinterpret_cast<const half4_t *>(up);
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++) b[j] = (4 * g + j < K) ? up[j] : (half_t)0;
        }
        const uint8_t *sb = packed + i * block_bytes + ((strip * SF_COLS) >> 3);
        sw = *reinterpret_cast<const uint4_t *>(sb + off_s);
    };
    // The (strip, block) pairs of this wave form one sequence over all its chunks; the sign and u loads run
    // NSETS - 1 pairs ahead, unconditionally (behind the last strip they repeat it).
    half4_t b_set[NSETS];
    uint4_t sw_set[NSETS];
#pragma unroll
    for (int k = 0; k < NSETS; k++) sw_set[k] = (uint4_t){0, 0, 0, 0};
    int pf_i = 0, pf_strip = first_strip;
    auto request = [&](half4_t &b, uint4_t &sw) {
        load_block(pf_i, min(pf_strip, strips - 1), b, sw);
        if (++pf_i == I) {
            pf_i = 0;
            pf_strip++;
        }
    };
#pragma unroll
    for (int k = 0; k + 1 < NSETS; k++) request(b_set[k], sw_set[k]);

    float4_t yacc[TT], acc[8];
#pragma unroll
    for (int tt = 0; tt < TT; tt++) yacc[tt] = (float4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < 8; s++) acc[s] = (float4_t){0.f, 0.f, 0.f, 0.f};
    const half_t *xfrag = xl + lm * xstride + 8 * g;   // token lm of a tile, columns 32 (s / 2) + 8 g + 4 (s % 2) .. + 3 of patch s

    // x and vt images of the chunk of strips that starts at s_begin (every thread of the workgroup arrives here together)
    auto stage = [&](int s_begin) {
        const int ns = min(sg, strips - s_begin);
        const int n0 = s_begin * SF_COLS;
        if (s_begin != first_strip) __syncthreads();   // everybody has finished with the previous images
        // x image: token rows beyond T are zero
        for (int idx = tid; idx < TT * 16 * ns * 16; idx += NT) {
            const int t = idx / (ns * 16), piece = idx % (ns * 16);
            half8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
            if (t < T) v = *reinterpret_cast<const half8_t *>(x + (int64_t)t * N + n0 + 8 * piece);
            *reinterpret_cast<half4_t *>(xl + t * xstride + 8 * piece) = (half4_t){v[0], v[1], v[2], v[3]};
        *reinterpret_cast<half4_t *>(xl + t * xstride + 8 * piece + 4) = (half4_t){v[4], v[5], v[6], v[7]};
        }
        // vt slices, four (strip, block) pairs per thread at a time so that their loads are in flight together
        for (int q0 = 0; q0 < ns * I; q0 += 8) {
            half8_t v[4];
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const int qi = min(q0 + k * 2 + spair, ns * I - 1), q = qi / I, i = qi - q * I;
                v[k] = (half8_t){0, 0, 0, 0, 0, 0, 0, 0};
                if (sr < K) v[k] = *reinterpret_cast<const half8_t *>(vt + ((int64_t)i * K + sr) * N + n0 + q * SF_COLS + 8 * sp);
            }
#pragma unroll
            for (int k = 0; k < 4; k++) {
                if (q0 + k * 2 + spair < ns * I) {
#pragma unroll
                    for (int e = 0; e < 8; e++) vl[(q0 + k * 2 + spair) * VBLOCK + (8 * sp + e) * VSTRIDE + sp * VGROUP_PAD + sr] = v[k][e];
                }
            }
        }
        __syncthreads();
    };

    // the pair being consumed: strip q of the current chunk, block i
    int i = 0, q = 0;
    auto consume = [&](const half4_t &b, const uint4_t &sw) {
        const half_t *vb = vl + (q * I + i) * VBLOCK + aoff;
        if (PEEL && i == 0)
            rebuild_block<true>(vb, b, sw, st, acc);
        else
            rebuild_block<false>(vb, b, sw, st, acc);
        if (++i < I) return;
        i = 0;
        // y[token, row] += x[token, these columns] . w[row, these columns], w rounded to fp16 as the dense path rounds it
        const half_t *xq = xfrag + q * SF_COLS;
#pragma unroll
        for (int s = 0; s < 8; s++) {
            const half4_t wf = {(half_t)acc[s][0], (half_t)acc[s][1], (half_t)acc[s][2], (half_t)acc[s][3]};
            if (!PEEL) acc[s] = (float4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int tt = 0; tt < TT; tt++) {
                const half4_t xf = *reinterpret_cast<const half4_t *>(xq + tt * 16 * xstride + 32 * (s >> 1) + 4 * (s & 1));
                yacc[tt] = __builtin_amdgcn_mfma_f32_16x16x16f16(xf, wf, yacc[tt], 0, 0, 0);
            }
        }
        q++;
    };
    for (int ch = 0; ch < n_chunk; ch++) {
        const int s_begin = first_strip + ch * sg;
        if (s_begin >= strips) break;                  // the same for every thread of the workgroup
        // Staging (loads behind branches, barriers) makes the compiler wait for every load in flight, so it stays
        // outside the loop over the pairs: once per chunk instead of once per pair.
        stage(s_begin);
        q = 0;
        const int n_pairs = min(sg, strips - s_begin) * I;
        for (int p = 0; p < n_pairs; p += NSETS) {
#pragma unroll
            for (int k = 0; k < NSETS; k++) {
                if (k > 0 && p + k >= n_pairs) break;
                request(b_set[(k + NSETS - 1) % NSETS], sw_set[(k + NSETS - 1) % NSETS]);   // the set consumed last
                consume(b_set[k], sw_set[k]);
            }
        }
        // the next chunk starts with set 0 again: turn the sets by what this chunk's pairs left over (the copies wait
        // for the requests in flight, as the staging of the next chunk does anyway)
        for (int r = n_pairs % NSETS; r > 0; r--) {
            const half4_t b0 = b_set[0];
            const uint4_t sw0 = sw_set[0];
#pragma unroll
            for (int k = 0; k + 1 < NSETS; k++) {
                b_set[k] = b_set[k + 1];
                sw_set[k] = sw_set[k + 1];
            }
            b_set[NSETS - 1] = b0;
            sw_set[NSETS - 1] = sw0;
        }
    }
    if (m0 + lm < M) {
#pragma unroll
        for (int tt = 0; tt < TT; tt++)
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const int t = 16 * tt + 4 * g + v;
                if (t < T) mat.part[((int64_t)cgroup * T + t) * M + m0 + lm] = yacc[tt][v];
            }
    }
}

// Column groups and strips per chunk of the walked kernel: two workgroups per CU (LDS), about two per CU in all.
// sign table, x image of tt token tiles, vt images of sg strips
size_t strip_lds(int I, int tt, int sg) {
    return (SIGN_LUT_HALVES + (size_t)sg * I * VBLOCK + (size_t)tt * 16 * (sg * SF_COLS + XPAD)) * sizeof(half_t);
}

struct WidePlan {
    int tt, sg, n_chunk, col_groups, row_tiles;
    size_t lds;
    bool worth;      // expected to beat rebuild + dense product
};
// Up to six token tiles two workgroups share a CU (122-128 registers); seven and eight tiles would need 133 and 159, one
// workgroup per CU, and lose to rebuild + dense kernel on every large shape.
constexpr int WIDE_MIN_T = 49, WIDE_MAX_T = 96;

WidePlan make_wide_plan(int I, int M, int N, int T) {
    WidePlan p;
    p.tt = (T + 15) / 16;
    p.row_tiles = (int)bs_cdiv(M, 128);
    const int strips = N / SF_COLS;
    p.sg = 0;
    for (int sg = 8; sg >= 1; sg >>= 1) {
        const size_t lds = strip_lds(I, p.tt, sg);
        if (lds * 2 <= 160 * 1024 || sg == 1) {
            p.sg = sg;
            p.lds = lds;
            break;
        }
    }
    const int chunks = (int)bs_cdiv(strips, p.sg);
    // as many column groups as fill the workgroup slots of the chip (two per CU) without a second round
    const int slots = 512;
    int cg = slots / p.row_tiles;
    if (cg > chunks) cg = chunks;
    if (cg < 1) cg = 1;
    p.n_chunk = (int)bs_cdiv(chunks, cg);
    p.col_groups = (int)bs_cdiv(chunks, p.n_chunk);
    // Measured against rebuild + vendor GEMM (8B layer shapes, layers alternating): per block both cost about the
    // same, but the walked kernel saves the round trip of the weight through memory, so it wins - by up to 1.3x -
    // wherever its workgroups fill the chip (1024 x 4096 with 8 blocks at 64 tokens 20 against 25 us, 4096 x 14336
    // 93 against 106) and loses where they do not (14336 x 4096, 448 workgroups for 512 slots: 90 against 74 us with
    // 6 blocks at 64 tokens, level with 3).  The exception is a matrix wider than tall with few blocks: the GEMM behind
    // its rebuild has few output tiles and a long inner dimension, and the walked kernel stays ahead at 448 workgroups
    // too (4096 x 14336 at 49 tokens: 50 against 60-66 us with 3 blocks, 71 against 78-84 with 6).
    const int grid = p.row_tiles * p.col_groups;
    // (up to one workgroup per CU nothing is uneven; beyond, the busiest CU holds a whole number of rounds of two)
    const double fill = grid <= slots / 2 ? 1.0 : (double)grid / (double)(bs_cdiv(grid, slots) * slots);
    p.worth = fill >= 0.95 || (M < N && I <= 6 && p.tt <= 5);
    return p;
}

template <int TT, bool K16>
int launch_wide_k(const WideMat &m, int grid, size_t lds, const half_t *x, int N, int K, int T, hipStream_t s) {
    static bs_lds_grant granted[BS_MAX_DEVICES];
    const int st = bs_allow_lds((const void *)strip_wide_kernel<TT, K16>, lds, granted);
    if (st != BS_OK) return st;
    strip_wide_kernel<TT, K16><<<grid, 512, lds, s>>>(m, x, N, K, T);
    BS_LAUNCH_CHECK();
    return BS_OK;
}
template <int TT>
int launch_wide(const WideMat &m, int grid, size_t lds, const half_t *x, int N, int K, int T, hipStream_t s) {
    return K == 16 ? launch_wide_k<TT, true>(m, grid, lds, x, N, K, T, s) : launch_wide_k<TT, false>(m, grid, lds, x, N, K, T, s);
}

struct StripPlan {
    int tt, sg, groups, gx, row_groups, rows_per_wg;
    size_t lds;
};

int token_tiles(int T) { return (T + 15) / 16; }


// Workgroups of 8 waves (two per CU): they share one vt image, so a CU holds 16 waves with half the
// LDS four-wave workgroups would need (at 16 blocks two of those, 8 waves, were all a CU could hold).
constexpr int STRIP_WAVES = 8;

// Strips per workgroup (a power of two up to 8) and row groups: of the choices that keep two
// workgroups on a CU and give every CU one, the one with the least work on the busiest CU -
// workgroups per CU x row steps per workgroup x strips per workgroup, which is what the rounding of
// rows to whole steps of 128 and of workgroups to whole CUs changes - and among equals the most
// strips (fewest partial sums).
StripPlan make_strip_plan(int I, int M, int N, int T) {
    StripPlan best;
    best.sg = 0;
    long best_cost = 0;
    const int tt = token_tiles(T), rs = 16 * STRIP_WAVES, cap = 16 / STRIP_WAVES;
    const int strips = N / SF_COLS;
    for (int sg = 8; sg >= 1; sg >>= 1) {
        StripPlan p;
        p.tt = tt;
        p.sg = sg;
        p.lds = strip_lds(I, tt, sg);
        if (sg > 1 && p.lds * cap > 160 * 1024) continue;
        if (sg > 1 && bs_cdiv(strips, sg) * bs_cdiv(M, rs) < 256) continue;
        int per_cu = (int)((160 * 1024) / p.lds);
        if (per_cu > cap) per_cu = cap;
        if (per_cu < 1) per_cu = 1;
        p.groups = (int)bs_cdiv(strips, sg);
        const int per_line = 8 / sg;
        p.gx = (int)bs_cdiv(p.groups, per_line) * per_line;
        int row_groups = (256 * per_cu) / p.gx;
        if (row_groups < 1) row_groups = 1;
        p.rows_per_wg = (int)bs_cdiv(bs_cdiv(M, row_groups), rs) * rs;
        p.row_groups = (int)bs_cdiv(M, p.rows_per_wg);
        const long cost = (long)bs_cdiv(p.gx * p.row_groups, 256) * (p.rows_per_wg / rs) * sg;
        if (best.sg == 0 || cost < best_cost) {
            best = p;
            best_cost = cost;
        }
    }
    return best;
}

template <int TT, int WAVES, bool K16>
int launch_ttw(const StripGroup &grp, int grid, size_t lds, const half_t *x, int N, int K, int T, hipStream_t s) {
    static bs_lds_grant granted[BS_MAX_DEVICES];
    const int st = bs_allow_lds((const void *)strip_forward_kernel<TT, WAVES, K16>, lds, granted);
    if (st != BS_OK) return st;
    strip_forward_kernel<TT, WAVES, K16><<<grid, 64 * WAVES, lds, s>>>(grp, x, N, K, T);
    BS_LAUNCH_CHECK();
    return BS_OK;
}

template <int TT>
int launch_tt(const StripGroup &grp, int grid, size_t lds, const half_t *x, int N, int K, int T, hipStream_t s) {
    return K == 16 ? launch_ttw<TT, STRIP_WAVES, true>(grp, grid, lds, x, N, K, T, s)
                   : launch_ttw<TT, STRIP_WAVES, false>(grp, grid, lds, x, N, K, T, s);
}

}  // namespace

// 49 tokens and more: the walked kernel (49..96 tokens, where its plan says it is worth it) or the panel kernel (up to
// BS_PANEL_MAX_T tokens); bs_set_prefill_kernel can pin either, or switch both off.
static int wide_partials(int I, int M, int N, int K, int T) {
    if (T > WIDE_MAX_T) return 0;
    // the walked kernel: 32-bit row offsets, and an LDS image of one strip that leaves room for two workgroups
    if ((int64_t)M * (N >> 3) >= ((int64_t)1 << 32) || (int64_t)M * K * 2 >= ((int64_t)1 << 32)) return 0;
    const WidePlan p = make_wide_plan(I, M, N, T);
    const bool worth = p.worth || bs_prefill_mode() == BS_PREFILL_WALKED;
    return (p.lds * 2 <= 160 * 1024 && worth && p.col_groups <= 1024) ? p.col_groups : 0;
}
// 1: walked kernel, 2: panel kernel, 0: neither (the weight is rebuilt)
static int wide_choice(int I, int M, int N, int K, int T) {
    const int mode = bs_prefill_mode();
    if (mode == BS_PREFILL_REBUILD) return 0;
    const bool walked = wide_partials(I, M, N, K, T) > 0, panel = bs_panel_partials(I, M, N, K, T) > 0;
    if (mode == BS_PREFILL_WALKED) return walked ? 1 : 0;
    if (mode == BS_PREFILL_PANEL) return panel ? 2 : 0;
    // Both take the shape: the walked kernel requests its sign words strip by strip (16 bytes per row and request, every
    // line eight times from L2), which costs more the more blocks there are and the more rows share a column range; the
    // panel kernel requests four strips at a time but pays two barriers and an LDS round trip of the weight tile per
    // strip.  Measured on the four 8B shapes, 2 to 8 blocks, 49 to 96 tokens: the panel kernel is ahead from 6 blocks
    // on the tall shapes (14336 x 4096: 78 against 80 us at 6 blocks, 91 against 101 at 8) and from 5 blocks above 80
    // tokens (214 against 221 us over the four layers at 6 blocks, 244 against 266 at 8); the walked kernel elsewhere
    // (by 10 to 25 % up to 4 blocks).
    if (walked && panel) return ((I >= 6 && M > N) || (T > 80 && I >= 5)) ? 2 : 1;
    return walked ? 1 : panel ? 2 : 0;
}

// Which of this family's kernels a forward of these dimensions runs: 0 none, 1 strip_forward_kernel (5..48 tokens),
// 2 strip_wide_kernel (the walked strips), 3 the panel kernel.
int bs_strip_kernel_choice(int I, int M, int N, int K, int T) {
    if (bs_strip_partials(I, M, N, K, T) == 0) return 0;
    if (T < WIDE_MIN_T) return 1;
    return wide_choice(I, M, N, K, T) == 1 ? 2 : 3;
}

// Partial sums per output (groups of strips) when this path takes the shape, else 0.
int bs_strip_partials(int I, int M, int N, int K, int T) {
    if (I < 1 || M < 1 || T < 1 || T > BS_PANEL_MAX_T || N % SF_COLS != 0) return 0;
    if ((int64_t)M * N >= ((int64_t)1 << 34)) return 0;
    if (T >= WIDE_MIN_T) {
        const int c = wide_choice(I, M, N, K, T);
        return c == 1 ? wide_partials(I, M, N, K, T) : c == 2 ? bs_panel_partials(I, M, N, K, T) : 0;
    }
    if (strip_lds(I, token_tiles(T), 1) > 160 * 1024) return 0;
    const StripPlan p = make_strip_plan(I, M, N, T);
    return p.groups <= 1024 ? p.groups : 0;
}

// One launch for n <= 4 matrices that read x: part[j] receives [bs_strip_partials(j), T, M[j]]
// floats; ssq (may be null) receives [bs_strip_partials(0), T] sums of squares of x.
int bs_launch_strip_group(int n, const uint8_t *const *packed, const half_t *const *u, const half_t *const *vt,
                          const int *I, const int *M, float *const *part, float *ssq, const half_t *x,
                          int N, int K, int T, hipStream_t s) {
    if (n < 1 || n > STRIP_MAX_GROUP || !bs_aligned(x, 16)) return BS_ERR_SHAPE;
    if (T >= WIDE_MIN_T) {
        // one matrix, no sums of squares: these kernels serve bs_forward's calls only
        if (n != 1 || ssq || bs_strip_partials(I[0], M[0], N, K, T) == 0) return BS_ERR_SHAPE;
        if (!bs_aligned(packed[0], 16) || !bs_aligned(vt[0], 16) || !bs_aligned(u[0], 8)) return BS_ERR_SHAPE;
        if (wide_choice(I[0], M[0], N, K, T) == 2) return bs_launch_panel(packed[0], u[0], vt[0], I[0], M[0], part[0], x, N, K, T, s);
        const WidePlan p = make_wide_plan(I[0], M[0], N, T);
        const WideMat m{packed[0], u[0], vt[0], part[0], I[0], M[0], p.sg, p.n_chunk, p.row_tiles};
        const int grid = p.row_tiles * p.col_groups;
        switch (p.tt) {
            case 4: return launch_wide<4>(m, grid, p.lds, x, N, K, T, s);
            case 5: return launch_wide<5>(m, grid, p.lds, x, N, K, T, s);
            default: return launch_wide<6>(m, grid, p.lds, x, N, K, T, s);
        }
    }
    StripGroup grp;
    grp.n = n;
    grp.ssq = ssq;
    size_t lds = 0;
    int slots = 0;
    for (int j = 0; j < n; j++) {
        if (bs_strip_partials(I[j], M[j], N, K, T) == 0) return BS_ERR_SHAPE;
        if (!bs_aligned(packed[j], 16) || !bs_aligned(vt[j], 16) || !bs_aligned(u[j], 8)) return BS_ERR_SHAPE;
        const StripPlan p = make_strip_plan(I[j], M[j], N, T);
        grp.m[j] = StripMat{packed[j], u[j], vt[j], part[j], I[j], M[j], p.sg, p.rows_per_wg, p.row_groups, slots};
        slots += (int)bs_cdiv(p.gx * p.row_groups, 8) * 8;
        if (p.lds > lds) lds = p.lds;
    }
    for (int j = n; j < STRIP_MAX_GROUP; j++) grp.m[j] = grp.m[0];
    return token_tiles(T) == 1 ? launch_tt<1>(grp, slots, lds, x, N, K, T, s) : token_tiles(T) == 2 ? launch_tt<2>(grp, slots, lds, x, N, K, T, s) : launch_tt<3>(grp, slots, lds, x, N, K, T, s);
}

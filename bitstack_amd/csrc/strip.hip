// Forward for a handful to a few dozen tokens on gfx950: the weight is rebuilt patch by
// patch in registers and multiplied by x at once; it never goes to memory.
//
//   part[strip, t, m] = sum_{n in strip} x[t, n] * fp16( sum_i s_i[m, n] * sum_r u_i[m, r] * vt_i[r, n] )
//
// Same decomposition as the weight rebuild (a workgroup owns a strip of 128 columns and
// a range of rows, the strip's slice of vt of ALL blocks staged transposed in LDS, per
// block one v_mfma_f32_16x16x16_f16 per 16 x 16 patch computed transposed, sign applied
// as bit 31 of 1.0f in one FMA).  When the last block of a 16-row step is in, a lane
// holds w[m0 + lm, 4 consecutive columns] of each patch - exactly the B operand of a
// second v_mfma_f32_16x16x16_f16 whose A operand is x[16 tokens, the same 4 columns]
// (read from an LDS copy of the strip's slice of x) and whose result is y[token, row]
// for this strip.  w is rounded to fp16 before that product, as it is when it is stored
// and multiplied by the dense kernel.  The strips' partial sums go to scratch
// [strip, T, M] (fp32); the reduce kernel of the decode path adds them in strip order
// and applies bias and epilogue.
//
// Cost per 16 x 16 patch and block: the same ~14 VALU operations as the rebuild, no store
// of w (two thirds of the rebuild's bytes) and no second pass that reads it back; the
// token count only adds one MFMA per patch and 16 tokens, after the last block.
#include "common.h"

namespace {

constexpr int SF_COLS = 128;    // columns per strip
constexpr int VSTRIDE = 16;     // halves per column of the vt image: the 16 ranks
constexpr int VGROUP_PAD = 4;   // extra halves after every 8 columns
constexpr int VBLOCK = SF_COLS * VSTRIDE + (SF_COLS / 8) * VGROUP_PAD;   // halves per block

// TT = token tiles of 16.  A workgroup takes `sg` (1, 2, 4 or 8) neighbouring strips at once:
// their vt slices are staged together, and per 16-row step the partial y of all of them
// is added up in registers, so scratch holds one partial per GROUP of strips and a lane
// reads sg * 16 consecutive sign bytes of its row.
template <int TT>
__global__ __launch_bounds__(256, 4) void strip_forward_kernel(
    const uint8_t *__restrict__ packed, const half_t *__restrict__ u, const half_t *__restrict__ vt,
    const half_t *__restrict__ x, float *__restrict__ part, int I, int M, int N, int K, int T, int sg,
    int rows_per_wg) {
    extern __shared__ __attribute__((aligned(16))) half_t lds[];
    const int xstride = sg * SF_COLS + 8;           // halves per token row of the x image
    half_t *xl = lds;                               // [TT * 16][xstride]
    half_t *vl = lds + TT * 16 * xstride;           // [sg][I][VBLOCK]

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lm = lane & 15, g = lane >> 4;
    // Slot order (128-byte line of sign bytes, row group, strip group within the line),
    // contiguous runs of slots per XCD: the 8 / sg groups that share a line meet in one L2.
    // gridDim.x counts strip groups padded to whole lines; slots beyond the last strip idle.
    int group, row_begin;
    {
        const int per_line = 8 / sg;
        const int nb = gridDim.x * gridDim.y, lin = blockIdx.x + gridDim.x * blockIdx.y;
        const int xcd = lin & 7, loc = lin >> 3, base = nb >> 3, rem = nb & 7;
        const int v = xcd * base + min(xcd, rem) + loc;
        const int rest = v / per_line;
        group = (rest / (int)gridDim.y) * per_line + v % per_line;
        row_begin = (rest % (int)gridDim.y) * rows_per_wg;
    }
    const int strips = N / SF_COLS;
    const int s_begin = group * sg;
    if (s_begin >= strips) return;
    const int ns = min(sg, strips - s_begin);       // strips this workgroup really has
    const int n0 = s_begin * SF_COLS;
    const int row_end = min(row_begin + rows_per_wg, M);
    const int64_t row_bytes = N >> 3;
    const int64_t block_bytes = (int64_t)M * row_bytes;

    const int sr = tid & 15, sp = tid >> 4;         // staging role: rank, piece of 8 columns
    const int sh_byte = 24 - 8 * g;                 // brings the lane's byte of a sign word to the top
    const int acol = 8 * (lm >> 2) + (lm & 3);
    const int aoff = acol * VSTRIDE + (lm >> 2) * VGROUP_PAD + 4 * g;

    auto load_block = [&](int i, int row, int q, half4_t &b, uint4_t &sw) {
        const half_t *up = u + ((int64_t)i * M + row) * K + 4 * g;
        if (K == 16) {
            b = *reinterpret_cast<const half4_t *>(up);
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++) b[j] = (4 * g + j < K) ? up[j] : (half_t)0;
        }
        sw = *reinterpret_cast<const uint4_t *>(packed + i * block_bytes + row * row_bytes + ((n0 + q * SF_COLS) >> 3));
    };
    half4_t b_cur, b_nxt;
    uint4_t sw_cur = {0, 0, 0, 0}, sw_nxt = {0, 0, 0, 0};
    if (row_begin + wave * 16 < row_end) load_block(0, min(row_begin + wave * 16 + lm, M - 1), 0, b_cur, sw_cur);

    // x image: token rows beyond T are zero
    for (int idx = tid; idx < TT * 16 * ns * 16; idx += 256) {
        const int t = idx / (ns * 16), piece = idx % (ns * 16);
        half8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
        if (t < T) v = *reinterpret_cast<const half8_t *>(x + (int64_t)t * N + n0 + 8 * piece);
        *reinterpret_cast<half8_t *>(xl + t * xstride + 8 * piece) = v;
    }
    // vt slices, four (strip, block) pairs at a time so that their loads are in flight together
    for (int q0 = 0; q0 < ns * I; q0 += 4) {
        half8_t v[4];
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const int qi = min(q0 + k, ns * I - 1), q = qi / I, i = qi - q * I;
            v[k] = (half8_t){0, 0, 0, 0, 0, 0, 0, 0};
            if (sr < K) v[k] = *reinterpret_cast<const half8_t *>(vt + ((int64_t)i * K + sr) * N + n0 + q * SF_COLS + 8 * sp);
        }
#pragma unroll
        for (int k = 0; k < 4; k++) {
            if (q0 + k < ns * I) {
#pragma unroll
                for (int e = 0; e < 8; e++) vl[(q0 + k) * VBLOCK + (8 * sp + e) * VSTRIDE + sp * VGROUP_PAD + sr] = v[k][e];
            }
        }
    }
    __syncthreads();

    // this lane's x fragments: token lm of a tile, columns 32 (s / 2) + 8 g + 4 (s % 2) .. + 3 of patch s
    const half_t *xfrag = xl + lm * xstride + 8 * g;

    for (int m0 = row_begin + wave * 16; m0 < row_end; m0 += 64) {
        const int row = min(m0 + lm, M - 1);
        float4_t yacc[TT];
#pragma unroll
        for (int tt = 0; tt < TT; tt++) yacc[tt] = (float4_t){0.f, 0.f, 0.f, 0.f};

        for (int q = 0; q < ns; q++) {
            float4_t acc[8];
#pragma unroll
            for (int s = 0; s < 8; s++) acc[s] = (float4_t){0.f, 0.f, 0.f, 0.f};

            for (int i = 0; i < I; i++) {
                // signs and u one block ahead, across strips and row steps
                if (i + 1 < I) load_block(i + 1, row, q, b_nxt, sw_nxt);
                else if (q + 1 < ns) load_block(0, row, q + 1, b_nxt, sw_nxt);
                else if (m0 + 64 < row_end) load_block(0, min(m0 + 64 + lm, M - 1), 0, b_nxt, sw_nxt);
                const uint4_t swc = sw_cur;         // bit 1 means +1: the product enters negated, times -1.0f
                const half_t *vb = vl + (q * I + i) * VBLOCK + aoff;
#pragma unroll
                for (int s = 0; s < 8; s++) {
                    const half_t *ap = vb + (32 * (s >> 1) + 4 * (s & 1)) * VSTRIDE + 4 * (s >> 1) * VGROUP_PAD;
                    const half4_t a = *reinterpret_cast<const half4_t *>(ap);
                    const float4_t p = __builtin_amdgcn_mfma_f32_16x16x16f16(a, b_cur, (float4_t){0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
                    const uint32_t t = swc[s >> 1] << (sh_byte + 4 * (s & 1));
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        const uint32_t sf = ((t << j) & 0x80000000u) | 0x3F800000u;
                        acc[s][j] = __builtin_fmaf(-p[j], __builtin_bit_cast(float, sf), acc[s][j]);
                    }
                }
                b_cur = b_nxt;
                sw_cur = sw_nxt;
            }

            // y[token, row] of this strip: D[token 4g + v, row lm] = sum_k x[token, col(k)] * w[row, col(k)]
            const half_t *xq = xfrag + q * SF_COLS;
#pragma unroll
            for (int s = 0; s < 8; s++) {
                const half4_t wf = {(half_t)acc[s][0], (half_t)acc[s][1], (half_t)acc[s][2], (half_t)acc[s][3]};
#pragma unroll
                for (int tt = 0; tt < TT; tt++) {
                    const half4_t xf = *reinterpret_cast<const half4_t *>(xq + tt * 16 * xstride + 32 * (s >> 1) + 4 * (s & 1));
                    yacc[tt] = __builtin_amdgcn_mfma_f32_16x16x16f16(xf, wf, yacc[tt], 0, 0, 0);
                }
            }
        }
        if (m0 + lm < M) {
#pragma unroll
            for (int tt = 0; tt < TT; tt++)
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    const int t = 16 * tt + 4 * g + v;
                    if (t < T) part[((int64_t)group * T + t) * M + m0 + lm] = yacc[tt][v];
                }
        }
    }
}

struct StripPlan {
    int tt, sg, groups, gx, row_groups, rows_per_wg;
    size_t lds;
};

int token_tiles(int T) { return T <= 16 ? 1 : 2; }

size_t strip_lds(int I, int tt, int sg) {
    return ((size_t)sg * I * VBLOCK + (size_t)tt * 16 * (sg * SF_COLS + 8)) * sizeof(half_t);
}

// Strips per workgroup: as many (a power of two up to 8) as keep three workgroups on a
// CU and a grid of at least one workgroup per CU; then as
// many row groups as fill the resident slots once.
StripPlan make_strip_plan(int I, int M, int N, int T) {
    StripPlan p;
    p.tt = token_tiles(T);
    const int strips = N / SF_COLS, cap = 4, want = 3;
    p.sg = 1;
    for (int sg = 8; sg > 1; sg >>= 1) {
        if (strip_lds(I, p.tt, sg) * want > 160 * 1024) continue;
        if (bs_cdiv(strips, sg) * bs_cdiv(M, 64) < 256) continue;
        p.sg = sg;
        break;
    }
    p.lds = strip_lds(I, p.tt, p.sg);
    int per_cu = (int)((160 * 1024) / p.lds);
    if (per_cu > cap) per_cu = cap;
    if (per_cu < 1) per_cu = 1;
    p.groups = (int)bs_cdiv(strips, p.sg);
    const int per_line = 8 / p.sg;
    p.gx = (int)bs_cdiv(p.groups, per_line) * per_line;
    int row_groups = (256 * per_cu) / p.gx;
    if (row_groups < 1) row_groups = 1;
    p.rows_per_wg = (int)bs_cdiv(bs_cdiv(M, row_groups), 64) * 64;
    p.row_groups = (int)bs_cdiv(M, p.rows_per_wg);
    return p;
}

template <int TT>
int launch_tt(const StripPlan &p, const uint8_t *packed, const half_t *u, const half_t *vt, const half_t *x,
              float *part, int I, int M, int N, int K, int T, hipStream_t s) {
    static size_t granted[BS_MAX_DEVICES] = {};
    const int st = bs_allow_lds((const void *)strip_forward_kernel<TT>, p.lds, granted);
    if (st != BS_OK) return st;
    dim3 grid(p.gx, p.row_groups);
    strip_forward_kernel<TT><<<grid, 256, p.lds, s>>>(packed, u, vt, x, part, I, M, N, K, T, p.sg, p.rows_per_wg);
    BS_LAUNCH_CHECK();
    return BS_OK;
}

}  // namespace

// Partial sums per output (groups of strips) when this path takes the shape, else 0.
int bs_strip_partials(int I, int M, int N, int K, int T) {
    (void)K;
    if (I < 1 || M < 1 || T < 1 || T > 32 || N % SF_COLS != 0) return 0;
    if ((int64_t)M * N >= ((int64_t)1 << 34)) return 0;
    if (strip_lds(I, token_tiles(T), 1) > 160 * 1024) return 0;
    const StripPlan p = make_strip_plan(I, M, N, T);
    return p.groups <= 1024 ? p.groups : 0;
}

// part[group of strips, t, m]: bs_strip_partials x T x M floats
int bs_launch_strip_partials(const uint8_t *packed, const half_t *u, const half_t *vt, const half_t *x,
                             float *part, int I, int M, int N, int K, int T, hipStream_t s) {
    if (bs_strip_partials(I, M, N, K, T) == 0) return BS_ERR_SHAPE;
    if (!bs_aligned(packed, 16) || !bs_aligned(vt, 16) || !bs_aligned(u, 8) || !bs_aligned(x, 16)) return BS_ERR_SHAPE;
    const StripPlan p = make_strip_plan(I, M, N, T);
    switch (p.tt) {
        case 1: return launch_tt<1>(p, packed, u, vt, x, part, I, M, N, K, T, s);
        default: return launch_tt<2>(p, packed, u, vt, x, part, I, M, N, K, T, s);
    }
}

// Forward for about a hundred to a few hundred tokens on gfx950: sign tiles are decoded into LDS and
// multiplied on the fp16 matrix cores at once; the rebuilt weight never goes to memory.
//
//   part[g, t, m] = sum_{n in column group g} x[t, n] * fp16( sum_i s_i[m, n] * sum_r u_i[m, r] * vt_i[r, n] )
//
// A workgroup of 8 waves owns 128 rows, all (up to 128) tokens and a run of 128-column strips.  Per strip:
//   rebuild   every wave rebuilds its 16 rows of the strip patch by patch, exactly as the weight
//             rebuild does (the strip's slice of vt of all blocks transposed in LDS, one
//             v_mfma_f32_16x16x16_f16 per 16 x 16 patch and block, the signs of a nibble looked up as
//             four halves of +-1.0 and multiplied in by a mixed-precision FMA, fp32 sums over the
//             blocks), rounds once to fp16 - the rounding point of the stored weight - and writes its
//             16 x 128 piece into a W tile [128 rows][128 columns] in LDS;
//   multiply  the eight waves tile the 128 x 128 outputs (32 tokens x 64 rows each) and run
//             y += x_tile . W_tile^T on v_mfma_f32_32x32x16_f16 with both operands read from LDS,
//             fp32 accumulators in registers for the whole run of strips.
// The x slice and the vt slice of the NEXT strip travel through registers meanwhile (vt is requested
// before the rebuild and stored behind it, x is requested before the product and stored behind it), so
// a strip costs two barriers and no exposed memory latency.  At the end the accumulators go to scratch
// [column group, T, M] (fp32) and the summing kernel of the decode path adds the groups in order, adds
// the bias and rounds.  Against rebuild + dense product this saves writing the weight (2 M N bytes) and
// reading it back, which is most of the memory traffic of a forward at these token counts; per block
// the arithmetic is the same.
#include "common.h"
#include "rebuild_shared.h"

#include <type_traits>

namespace {

constexpr int PN_ROWS = 128;            // rows per workgroup: 16 per wave
constexpr int PN_LD = SF_COLS + 8;      // halves per row of the W and x tiles (rows 16 bytes apart in the banks)

struct PanelMat {
    const uint8_t *packed;
    const half_t *u, *vt;
    float *part;
    int I, M, row_tiles, strips_per_group;
};

constexpr int PN_MAXB = 8;              // most blocks: their u rows and sign words live in registers
// Tokens per workgroup.  (A 256-token instantiation - 64 accumulator registers per lane instead of 32 - spills over a
// hundred registers next to the resident sign words and u rows, and without them it did not beat rebuild + dense
// product on the tall shapes; above 128 tokens the weight is rebuilt once and multiplied by the dense kernel.)
constexpr int PN_TOKENS = 128;
static_assert(PN_TOKENS == BS_PANEL_MAX_T, "one token block per call");

// BT: tokens per workgroup.  K16 as in the rebuild kernel.
template <int BT, bool K16>
__global__ __launch_bounds__(512, 2) void panel_forward_kernel(const PanelMat mat, const half_t *__restrict__ x, int N, int K, int T) {
    constexpr int TA = BT / 128;            // 32-token A fragments per wave (its tile is BT / 4 tokens x 64 rows)
    constexpr int XP = BT / 32;             // 16-byte x pieces a thread carries for the next strip
    constexpr int NV = 4;                   // 16-byte vt pieces a thread carries for the next strip (four ranks of one block)
    static_assert(PN_MAXB == 8, "one wave per block stages vt");
    extern __shared__ __attribute__((aligned(128))) half_t lds_all[];
    const int I = mat.I, M = mat.M;
    half_t *const vl = lds_all + SIGN_LUT_HALVES;       // [I][VBLOCK]
    half_t *const wl = vl + I * VBLOCK;                 // [128][PN_LD]
    half_t *const xl = wl + PN_ROWS * PN_LD;            // [BT][PN_LD]
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lm = lane & 15, g = lane >> 4;
    // Workgroups are dealt round-robin to the 8 XCDs; every XCD gets a contiguous run of (column group, row tile)
    // slots with the row tile fastest, so the workgroups that read the same slices of x and vt share an L2.
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
    const int strips = N / SF_COLS;
    const int first_strip = cgroup * mat.strips_per_group;
    const int end_strip = min(first_strip + mat.strips_per_group, strips);
    if (first_strip >= end_strip) return;               // (the same for every thread of the workgroup)
    const int64_t row_bytes = N >> 3;
    const int64_t block_bytes = (int64_t)M * row_bytes;

    const SignTable st = make_sign_table(lds_all, tid, g);
    const int acol = 8 * (lm >> 2) + (lm & 3);
    const int aoff = acol * VSTRIDE + (lm >> 2) * VGROUP_PAD + 4 * g;

    // ---- rebuild role: rows m0 .. m0 + 15 of the workgroup's tile, lane (g, lm) = (rank quad / column byte, row) ----
    const int m0 = rt * PN_ROWS + wave * 16;
    const int row = min(m0 + lm, M - 1);
    // The rows never change, so the u rows of all blocks are loaded once (blocks beyond I repeat the last one, unused).
    half4_t ub[PN_MAXB];
#pragma unroll
    for (int i = 0; i < PN_MAXB; i++) {
        const half_t *urow = u + ((int64_t)min(i, I - 1) * M + row) * K;
        if (K16) {
            ub[i] = *reinterpret_cast<const half4_t *>(urow + 4 * g);
        } else {
            // (ranks beyond K repeat rank K - 1 and are zeroed: no load outside the row)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const half_t val = urow[min(4 * g + j, K - 1)];
                ub[i][j] = (4 * g + j < K) ? val : (half_t)0;
            }
        }
    }
    // Sign words, FOUR STRIPS PER INSTRUCTION: lane group g loads the 16 bytes of strip 4 Q + g of its row (64
    // consecutive bytes of the row per instruction), for every block, and keeps them for the four strips of quad Q; the
    // strip being rebuilt fetches its words from the group that holds them with four cross-lane reads.  Loaded strip
    // by strip, all four groups requested the same 16 bytes, every instruction touched 16 different 128-byte lines for
    // 16 bytes each, and every line came from L2 again for each of its eight strips: eight times the sign bytes in
    // line traffic, which was half of this kernel's time.
    uint4_t sq[PN_MAXB];
    const uint32_t off_s = (uint32_t)row * (uint32_t)row_bytes;
    auto request_signs = [&](int quad) {
        const int strip = min(4 * quad + g, strips - 1);
        const uint8_t *sb = packed + ((strip * SF_COLS) >> 3) + off_s;
#pragma unroll
        for (int i = 0; i < PN_MAXB; i++) sq[i] = *reinterpret_cast<const uint4_t *>(sb + (int64_t)min(i, I - 1) * block_bytes);
    };
    auto sign_words = [&](const uint4_t &qd, int sel) {
        const int from = (16 * sel + lm) * 4;
        uint4_t r;
#pragma unroll
        for (int d = 0; d < 4; d++) r[d] = (uint32_t)__builtin_amdgcn_ds_bpermute(from, (int)qd[d]);
        return r;
    };
    request_signs(first_strip >> 2);

    // ---- staging roles ---------------------------------------------------------------------------------
    // vt: thread = (piece sp of 8 columns, rank quad rq, block `side`): four 16-byte loads (ranks 4 rq .. 4 rq + 3 of
    // the piece), transposed in registers, eight 8-byte stores into the image [column][rank] - a quarter of the LDS
    // instructions of storing rank by rank, two bytes at a time.
    const int sp = tid & 15, rq = (tid >> 4) & 3, side = tid >> 6;
    half8_t vpre[NV];
    auto request_vt = [&](int strip) {
        const half_t *vb = vt + (int64_t)min(side, I - 1) * K * N + strip * SF_COLS + 8 * sp;
#pragma unroll
        for (int k = 0; k < NV; k++) vpre[k] = *reinterpret_cast<const half8_t *>(vb + (int64_t)min(4 * rq + k, K - 1) * N);
    };
    auto store_vt = [&]() {
        if (side < I) {
            half_t *dst = vl + side * VBLOCK + 8 * sp * VSTRIDE + sp * VGROUP_PAD + 4 * rq;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                half4_t o;
#pragma unroll
                for (int k = 0; k < 4; k++) o[k] = (4 * rq + k < K) ? vpre[k][e] : (half_t)0;
                *reinterpret_cast<half4_t *>(dst + e * VSTRIDE) = o;
            }
        }
    };
    // x: thread = (piece xp of 8 columns, token row tid / 16 + 32 k); token rows beyond T are zero
    const int xp = tid & 15, xt = tid >> 4;
    half8_t xpre[XP];
    auto request_x = [&](int strip) {
        const int n0 = strip * SF_COLS;
#pragma unroll
        for (int k = 0; k < XP; k++) {
            const int t = xt + 32 * k;
            xpre[k] = *reinterpret_cast<const half8_t *>(x + (int64_t)min(t, T - 1) * N + n0 + 8 * xp);
        }
    };
    auto store_x = [&]() {
#pragma unroll
        for (int k = 0; k < XP; k++) {
            const int t = xt + 32 * k;
            half8_t v = xpre[k];
            if (t >= T) v = (half8_t){0, 0, 0, 0, 0, 0, 0, 0};
            *reinterpret_cast<half8_t *>(xl + t * PN_LD + 8 * xp) = v;
        }
    };

    // ---- multiply role: tokens wt * BT / 4 .., rows wr * 64 .. of the workgroup's tile -----------------------
    const int wt = wave & 3, wr = wave >> 2;
    const int l32 = lane & 31, kh = lane >> 5;
    const half_t *xa = xl + (wt * (BT / 4) + l32) * PN_LD + 8 * kh;
    const half_t *wb = wl + (wr * 64 + l32) * PN_LD + 8 * kh;
    float16_t yacc[TA][2];
#pragma unroll
    for (int a = 0; a < TA; a++)
#pragma unroll
        for (int b = 0; b < 2; b++)
#pragma unroll
            for (int v = 0; v < 16; v++) yacc[a][b][v] = 0.f;

    // ---- first strip's images ---------------------------------------------------------------------------
    request_vt(first_strip);
    request_x(first_strip);
    store_vt();
    store_x();
    __syncthreads();

    float4_t acc[8];
    // One strip: rebuild (blocks written out, so that every register array is indexed by constants), W tile, product.
    // RELOAD: this strip is the last of its quad (or of the run): every block's sign words are requested for the next
    // quad right behind their last use.  The two versions are separate code, chosen per strip: a load behind a branch
    // inside the block loop would make the compiler wait for every load in flight where the paths join.
    auto strip_body = [&](int strip, bool more, auto reload_tag) {
        constexpr bool RELOAD = decltype(reload_tag)::value;
        request_vt(more ? strip + 1 : strip);           // lands while this strip is rebuilt
        const int sel = strip & 3;
        const int next_quad = (strip + 1) >> 2;
        const uint8_t *sb_next = packed + ((min(4 * next_quad + g, strips - 1) * SF_COLS) >> 3) + off_s;
#pragma unroll
        for (int i = 0; i < PN_MAXB; i++) {
            if (i < I) {
                const uint4_t sw = sign_words(sq[i], sel);
                const half_t *vb = vl + i * VBLOCK + aoff;
                if (i == 0)
                    rebuild_block<true>(vb, ub[i], sw, st, acc);
                else
                    rebuild_block<false>(vb, ub[i], sw, st, acc);
            }
            if (RELOAD) sq[i] = *reinterpret_cast<const uint4_t *>(sb_next + (int64_t)min(i, I - 1) * block_bytes);
        }
        // one rounding to fp16, as the stored weight has it; lane (g, lm) holds columns 32 q + 8 g .. + 7 of row lm
        {
            half_t *wrow = wl + (wave * 16 + lm) * PN_LD + 8 * g;
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const half8_t o = {(half_t)acc[2 * q][0], (half_t)acc[2 * q][1], (half_t)acc[2 * q][2], (half_t)acc[2 * q][3],
                                   (half_t)acc[2 * q + 1][0], (half_t)acc[2 * q + 1][1], (half_t)acc[2 * q + 1][2], (half_t)acc[2 * q + 1][3]};
                *reinterpret_cast<half8_t *>(wrow + 32 * q) = o;
            }
        }
        __syncthreads();                                // the W tile is complete; nobody reads the vt image any more
        if (more) store_vt();
        request_x(more ? strip + 1 : strip);            // lands while this strip is multiplied
        // ---- y += x_tile . W_tile^T ----
#pragma unroll
        for (int ks = 0; ks < SF_COLS / 16; ks++) {
            half8_t fa[TA], fb[2];
#pragma unroll
            for (int a = 0; a < TA; a++) fa[a] = *reinterpret_cast<const half8_t *>(xa + a * 32 * PN_LD + 16 * ks);
#pragma unroll
            for (int b = 0; b < 2; b++) fb[b] = *reinterpret_cast<const half8_t *>(wb + b * 32 * PN_LD + 16 * ks);
#pragma unroll
            for (int a = 0; a < TA; a++)
#pragma unroll
                for (int b = 0; b < 2; b++) yacc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[a], fb[b], yacc[a][b], 0, 0, 0);
        }
        __syncthreads();                                // x and W tiles are free; the next vt image is in place
        if (more) store_x();                            // (visible to the product behind the next barrier)
    };
    for (int strip = first_strip; strip < end_strip; strip++) {
        const bool more = strip + 1 < end_strip;
        if ((strip & 3) == 3 && more)
            strip_body(strip, more, std::true_type{});
        else
            strip_body(strip, more, std::false_type{});
    }

    // ---- partial sums: D[token 8 (v / 4) + 4 kh + v % 4, row l32] of every 32 x 32 tile ----------------------
    float *part = mat.part + (int64_t)cgroup * T * M;
#pragma unroll
    for (int a = 0; a < TA; a++)
#pragma unroll
        for (int b = 0; b < 2; b++) {
            const int m = rt * PN_ROWS + wr * 64 + b * 32 + l32;
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int t = wt * (BT / 4) + a * 32 + 8 * (v >> 2) + 4 * kh + (v & 3);
                if (t < T && m < M) part[(int64_t)t * M + m] = yacc[a][b][v];
            }
        }
}

size_t panel_lds(int I, int bt) {
    return (SIGN_LUT_HALVES + (size_t)I * VBLOCK + (size_t)PN_ROWS * PN_LD + (size_t)bt * PN_LD) * sizeof(half_t);
}

struct PanelPlan {
    int bt, row_tiles, col_groups, strips_per_group;
    size_t lds;
    bool ok;
};

PanelPlan make_panel_plan(int I, int M, int N, int K, int T) {
    PanelPlan p;
    p.ok = false;
    p.bt = PN_TOKENS;
    p.row_tiles = (int)bs_cdiv(M, PN_ROWS);
    p.lds = panel_lds(I, p.bt);
    p.col_groups = p.strips_per_group = 0;
    if (I < 1 || I > PN_MAXB || T < 1 || T > BS_PANEL_MAX_T || N % SF_COLS != 0 || p.lds > 160 * 1024) return p;
    // the tiled addressing keeps a block's u and sign rows within 32-bit byte offsets
    if ((int64_t)M * (N >> 3) >= ((int64_t)1 << 32) || (int64_t)M * K * 2 >= ((int64_t)1 << 32)) return p;
    const int strips = N / SF_COLS;
    // one workgroup per CU (LDS): as many column groups as fill the chip, whole quads of strips (the 64 bytes of a
    // row one sign load brings) where the columns allow it, at most one group per strip
    int cg = 256 / p.row_tiles;
    if (cg > strips) cg = strips;
    if (cg < 1) cg = 1;
    p.strips_per_group = (int)bs_cdiv(strips, cg);
    if (p.strips_per_group > 4) p.strips_per_group = (int)bs_cdiv(p.strips_per_group, 4) * 4;
    p.col_groups = (int)bs_cdiv(strips, p.strips_per_group);
    p.ok = p.col_groups <= 1024;
    return p;
}

template <int BT, bool K16>
int launch_panel_k(const PanelMat &m, int grid, size_t lds, const half_t *x, int N, int K, int T, hipStream_t s) {
    static bs_lds_grant granted[BS_MAX_DEVICES];
    const int st = bs_allow_lds((const void *)panel_forward_kernel<BT, K16>, lds, granted);
    if (st != BS_OK) return st;
    panel_forward_kernel<BT, K16><<<grid, 512, lds, s>>>(m, x, N, K, T);
    BS_LAUNCH_CHECK();
    return BS_OK;
}

template <int BT>
int launch_panel(const PanelMat &m, int grid, size_t lds, const half_t *x, int N, int K, int T, hipStream_t s) {
    return K == 16 ? launch_panel_k<BT, true>(m, grid, lds, x, N, K, T, s) : launch_panel_k<BT, false>(m, grid, lds, x, N, K, T, s);
}

}  // namespace

// Column groups (partial sums per output) when the panel kernel takes the shape, else 0.
int bs_panel_partials(int I, int M, int N, int K, int T) {
    const PanelPlan p = make_panel_plan(I, M, N, K, T);
    return p.ok ? p.col_groups : 0;
}

// part receives [bs_panel_partials, T, M] floats.
int bs_launch_panel(const uint8_t *packed, const half_t *u, const half_t *vt, int I, int M, float *part, const half_t *x,
                    int N, int K, int T, hipStream_t s) {
    const PanelPlan p = make_panel_plan(I, M, N, K, T);
    if (!p.ok || !bs_aligned(x, 16) || !bs_aligned(packed, 16) || !bs_aligned(vt, 16) || !bs_aligned(u, 8)) return BS_ERR_SHAPE;
    const PanelMat m{packed, u, vt, part, I, M, p.row_tiles, p.strips_per_group};
    const int grid = p.row_tiles * p.col_groups;
    return launch_panel<PN_TOKENS>(m, grid, p.lds, x, N, K, T, s);
}

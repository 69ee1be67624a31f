// Dense fp16 contraction y[T, M] = x[T, N] @ w[M, N]^T (+ bias) on gfx950 MFMA.
//
// Both operands are contiguous along the contracted index N, which is what
// v_mfma_f32_32x32x16_f16 wants: a lane supplies eight consecutive k of one
// row (A = tokens) or one column (B = features), i.e. one 16-byte read per
// fragment.
//
// More than 128 tokens: linear_f16_kernel, WT x WF waves of AT x AF MFMA tiles each,
// k-steps of GK columns through two LDS buffers; rows are padded by 8 halves so that
// the lanes served per LDS cycle hit disjoint banks.  Four shapes are instantiated:
// 256 x 256 (8 waves of 128 x 64; GK = 64 with two register sets of pieces in flight when N % 64 == 0 - a row's 128
// bytes of a k-step are one cache line, fetched once; GK = 32 took every line from L2 twice, the halves a step apart and
// the L1 too small to keep them - else GK = 32 with three sets) and 128 x 256 (8 waves of 64 x 64) for
// grids that cover the chip, 128 x 128 and 64 x 64 (4 waves, two workgroups per CU,
// the latter with GK = 128: half as many barriers) for the smaller ones; the launcher
// takes the largest tile whose grid still has about 160 workgroups.
// The loop is software-pipelined at three levels, all through registers:
//   - global requests run NS k-steps ahead through NS register sets (four where the registers allow it: the
//     kernel waits for requests more than for anything else, and a fourth set is worth 3 to 13 %; five and six were
//     no better; two for the 256 x 256 tile in k-steps of 64), all of them unconditional buffer loads: descriptor,
//     32-bit lane offset, scalar k offset;
//   - the LDS writes of step s + 1 and the requests of step s + NS are cut into one
//     portion per MFMA group instead of one burst per step;
//   - MFMA fragments are read from LDS one group ahead of use, the first group of the
//     next step right behind the barrier.
// One barrier per step.  On this part LDS takes b128 reads at about 460 B/ns per CU
// and b128 writes at about 165 B/ns (independent of the lane-to-address map as long as
// rows are padded), global requests at 64 B per clock: with 64 x 64 per-wave tiles the
// LDS time equals the MFMA time, which is what the larger tiles are for.  Measured dead
// ends: 128 x 128 per-wave tiles with one wave per SIMD (nothing covers a wait), a
// per-workgroup rotation of the k order (less sharing in L2), 16-wave workgroups, requests
// that write LDS directly (global_load_lds_dwordx4: same time per step).
// 33..128 tokens use narrower workgroups of the same kernel (more workgroups for
// the few token rows); up to 32 tokens: linear_skinny_kernel (below).
#include "common.h"
#include <type_traits>
#include <utility>

namespace {

// Compile-time loop (the index is a constant expression inside the body).
template <class F, int... Is>
__device__ __forceinline__ void static_for_impl(F &&f, std::integer_sequence<int, Is...>) {
    (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F &&f) {
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// LDS rows of a k-step.  GK = 32: 64-byte rows with no padding, the four 16-byte pieces of a
// row XOR-ed with bits 2..3 of the row number - staging writes (four lanes per row, rows 64 bytes
// apart) and fragment reads (sixteen rows, one piece each) then both spread over all banks;
// with padded rows the writes of the 256 x 256 kernel conflicted (SQ_LDS_BANK_CONFLICT about a
// tenth of its cycles).  Wider steps: rows padded by 8 halves (no conflicts measured).
__host__ __device__ constexpr bool lds_swizzled(int gk) { return gk == 32; }
__host__ __device__ constexpr int lds_stride(int gk) { return lds_swizzled(gk) ? gk : gk + 8; }

template <int WT, int WF, int AT, int AF, int GK, bool KTAIL, int NS = 3>
__global__ __launch_bounds__(64 * WT * WF) void linear_f16_kernel(
    const half_t *__restrict__ x, const half_t *__restrict__ w, const half_t *__restrict__ bias,
    half_t *__restrict__ y, int T, int M, int N) {
    constexpr int THREADS = 64 * WT * WF;
    constexpr int BT = WT * AT * 32, BF = WF * AF * 32;      // workgroup tile: tokens x features
    constexpr int ROWS = BT + BF;                            // LDS rows per buffer (x rows, then w rows)
    constexpr int PPR = GK / 8;                              // 16-byte pieces per row and k-step
    constexpr int LSTRIDE = lds_stride(GK);                  // halves per LDS row
    constexpr bool SWZ = lds_swizzled(GK);
    constexpr int JX = BT * PPR / THREADS, JW = BF * PPR / THREADS;   // pieces per thread: x rows, w rows
    static_assert(BT * PPR % THREADS == 0 && BF * PPR % THREADS == 0, "every thread stages whole pieces");
    constexpr int PER_THREAD = JX + JW;
    extern __shared__ __attribute__((aligned(16))) half_t lds_raw[];
    half_t (*lds)[ROWS * LSTRIDE] = reinterpret_cast<half_t (*)[ROWS * LSTRIDE]>(lds_raw);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int t0 = blockIdx.y * BT, m0 = blockIdx.x * BF;
    const int wt = (wave / WF) * (AT * 32), wf = (wave % WF) * (AF * 32);
    const int l32 = lane & 31, kh = lane >> 5;

    // Loader role.  Piece j of a thread is row tid / PPR + (THREADS / PPR) * j of the x
    // tile (j < JX) or of the w tile, 16-byte piece tid % PPR.  Addresses are a
    // workgroup-uniform pointer (tile origin + k-step, scalar registers) plus a 32-bit
    // per-thread byte offset; rows beyond T or M repeat the last row (their outputs are
    // never stored), so no load in the main loop is conditional.
    const char *xt = reinterpret_cast<const char *>(x + (int64_t)t0 * N);
    const char *wt_ = reinterpret_cast<const char *>(w + (int64_t)m0 * N);
    const int lrow = tid / PPR, lpiece = tid % PPR;
    // raw buffer descriptors over the two tile origins (no stride, no range limit short of 4 GiB: offsets are checked
    // by construction - rows are clamped to the tile, k-steps to the contracted range)
    const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc((void *)xt, 0, -1, 0x00020000);
    const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc((void *)wt_, 0, -1, 0x00020000);
    uint32_t off[PER_THREAD];
    int dst[PER_THREAD];
#pragma unroll
    for (int j = 0; j < PER_THREAD; j++) {
        const bool isx = j < JX;
        const int r = lrow + (THREADS / PPR) * (isx ? j : j - JX);
        const int rr = isx ? min(r, T - 1 - t0) : min(r, M - 1 - m0);
        off[j] = (uint32_t)rr * (uint32_t)N * 2u + 16u * lpiece;
        dst[j] = ((isx ? 0 : BT) + r) * LSTRIDE + 8 * (SWZ ? (lpiece ^ ((r >> 2) & 3)) : lpiece);
    }

    float16_t acc[AT][AF];
#pragma unroll
    for (int a = 0; a < AT; a++)
#pragma unroll
        for (int b = 0; b < AF; b++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[a][b][v] = 0.f;

    const int steps = (N + GK - 1) / GK;
    // NS register sets: while step s is multiplied, the pieces of step s + 1 are in one set
    // (landed, on their way to LDS) and those of the steps up to s + NS in flight into the others.
    // Every request is unconditional (past the end the last step is requested again), so
    // the compiler's count of outstanding loads is exact and a wait for one set never
    // drains the other.  KTAIL (N not a multiple of GK): pieces beyond column N are read
    // from column 0 instead and replaced by zeros.
    uint4_t stage[NS][PER_THREAD];
    // part `part` of `parts` of the pieces of one step (the whole step: 0 of 1)
    auto fetch = [&](auto setc, int step_, auto partc, auto partsc) {
        constexpr int set = decltype(setc)::value, part = decltype(partc)::value, parts = decltype(partsc)::value;
        constexpr int j0 = part * PER_THREAD / parts, j1 = (part + 1) * PER_THREAD / parts;
        const int step = min(step_, steps - 1);
        if constexpr (KTAIL) {
            const bool in = step * GK + 8 * lpiece < N;              // N % 8 == 0: a piece is all in or all out
            const uint32_t koff = in ? (uint32_t)step * (GK * 2) : 0u - 16u * lpiece;
#pragma unroll
            for (int j = j0; j < j1; j++) {
                const uint4_t v = *reinterpret_cast<const uint4_t *>((j < JX ? xt : wt_) + (off[j] + koff));
                stage[set][j] = in ? v : (uint4_t){0, 0, 0, 0};
            }
        } else {
            // buffer loads: descriptor (tile origin) + 32-bit lane offset + scalar k offset - no 64-bit address arithmetic
            // per request (4-7 % of the kernel's time with flat global loads)
            const int koff = step * (GK * 2);
#pragma unroll
            for (int j = j0; j < j1; j++)
                stage[set][j] = __builtin_amdgcn_raw_buffer_load_b128(j < JX ? rx : rw, (int)off[j], koff, 0);
        }
    };
    // part `part` of `parts` of a register set goes to LDS (the whole set: 0 of 1)
    auto stash = [&](auto setc, int buf, auto partc, auto partsc) {
        constexpr int set = decltype(setc)::value, part = decltype(partc)::value, parts = decltype(partsc)::value;
#pragma unroll
        for (int j = part * PER_THREAD / parts; j < (part + 1) * PER_THREAD / parts; j++)
            *reinterpret_cast<uint4_t *>(&lds[buf][dst[j]]) = stage[set][j];
    };
    // Fragments travel through two register sets as well: the LDS reads of sub-step
    // kk + 1 are issued before the MFMAs of sub-step kk, and those of the next step's
    // first sub-step right after the barrier, before the MFMAs of this step's last one
    // (whose fragments were read before the barrier, so the buffer is free to be
    // overwritten).  No MFMA waits for an LDS read issued just before it.
    constexpr int NK = GK / 16;
    static_assert(NK % 2 == 0, "the fragment sets alternate with a period of two sub-steps");
    half8_t fa[2][AT], fb[2][AF];
    const int swz = (l32 >> 2) & 3;             // wt, wf and the tile offsets are multiples of 32: only the lane's row counts
    auto load_frags = [&](auto setc, int buf, int kk) {
        constexpr int set = decltype(setc)::value;
        const half_t *xs = &lds[buf][0], *ws = &lds[buf][BT * LSTRIDE];
#pragma unroll
        for (int j = 0; j < AT; j++)
            fa[set][j] = *reinterpret_cast<const half8_t *>(xs + (wt + 32 * j + l32) * LSTRIDE + (SWZ ? 8 * ((2 * kk + kh) ^ swz) : 16 * kk + 8 * kh));
#pragma unroll
        for (int j = 0; j < AF; j++)
            fb[set][j] = *reinterpret_cast<const half8_t *>(ws + (wf + 32 * j + l32) * LSTRIDE + (SWZ ? 8 * ((2 * kk + kh) ^ swz) : 16 * kk + 8 * kh));
    };
    auto mfmas = [&](auto setc) {
        constexpr int set = decltype(setc)::value;
#pragma unroll
        for (int ai = 0; ai < AT; ai++)
#pragma unroll
            for (int bi = 0; bi < AF; bi++)
                acc[ai][bi] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[set][ai], fb[set][bi], acc[ai][bi], 0, 0, 0);
    };
    using S0 = std::integral_constant<int, 0>;
    using S1 = std::integral_constant<int, 1>;
    // step s reads LDS buffer s & 1; its pieces travelled through register set s & 1
    // Neither the requests for step s + 2 nor the LDS writes of step s + 1 (requested a
    // step ago) are issued in one burst - a wave that queues six or more 1 KB requests
    // blocks on the address unit and every wave of the workgroup does so at the same
    // time, right after the barrier, with the matrix pipe idle.  Both are cut into
    // portions, one per group of MFMAs, issued together with the fragment reads in front
    // of the group.  Nobody reads the other LDS buffer between the previous barrier and
    // the next one, so it can be written all along the step.
    using PF = std::integral_constant<int, NK>;
    using PS = std::integral_constant<int, NK - 1>;
    using S2 = std::integral_constant<int, 2>;
    auto one_step = [&](auto cur, auto nxt, auto bufc, int step) {
        constexpr int buf = decltype(bufc)::value;
        static_for<NK / 2>([&](auto hc) {
            constexpr int kk = 2 * decltype(hc)::value;
            fetch(cur, step + NS, std::integral_constant<int, kk>{}, PF{});   // set `cur` was emptied into LDS a step ago
            load_frags(S1{}, buf, kk + 1);
            stash(nxt, buf ^ 1, std::integral_constant<int, kk>{}, PS{});    // after the last step: a copy nobody reads
            __builtin_amdgcn_sched_barrier(0);
            mfmas(S0{});
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (kk + 2 < NK) {
                fetch(cur, step + NS, std::integral_constant<int, kk + 1>{}, PF{});
                load_frags(S0{}, buf, kk + 2);
                stash(nxt, buf ^ 1, std::integral_constant<int, kk + 1>{}, PS{});
                __builtin_amdgcn_sched_barrier(0);
                mfmas(S1{});
                __builtin_amdgcn_sched_barrier(0);
            }
        });
        __syncthreads();
        fetch(cur, step + NS, std::integral_constant<int, NK - 1>{}, PF{});
        load_frags(S0{}, buf ^ 1, 0);
        __builtin_amdgcn_sched_barrier(0);
        mfmas(S1{});
        __builtin_amdgcn_sched_barrier(0);
    };

    // step s: its pieces travel through register set s % NS and are multiplied out of LDS buffer s % 2; the loop is
    // written out over one period of both, so that every set and buffer index is a constant
    static_for<NS>([&](auto kc) { fetch(kc, decltype(kc)::value, S0{}, S1{}); });
    stash(S0{}, 0, S0{}, S1{});
    __syncthreads();
    load_frags(S0{}, 0, 0);
    constexpr int PERIOD = NS % 2 == 0 ? NS : 2 * NS;
    for (int step = 0; step < steps; step += PERIOD) {
        static_for<PERIOD>([&](auto kc) {
            constexpr int k = decltype(kc)::value;
            if (k == 0 || step + k < steps)
                one_step(std::integral_constant<int, k % NS>{}, std::integral_constant<int, (k + 1) % NS>{},
                         std::integral_constant<int, k % 2>{}, step + k);
        });
    }

    // D[token, feature]: lane holds feature l32, tokens 8 * (v / 4) + 4 * kh + v % 4
#pragma unroll
    for (int bi = 0; bi < AF; bi++) {
        const int m = m0 + wf + 32 * bi + l32;
        if (m >= M) continue;
        const float bv = bias ? (float)bias[m] : 0.f;
#pragma unroll
        for (int ai = 0; ai < AT; ai++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int t = t0 + wt + 32 * ai + 8 * (v >> 2) + 4 * kh + (v & 3);
                if (t < T) y[(int64_t)t * M + m] = (half_t)(acc[ai][bi][v] + bv);
            }
    }
}

// Few tokens (<= 32): the job is to stream w once at memory speed, so nothing is
// shared through LDS.  A workgroup owns 32 features; its KS waves split the
// contracted range, each wave reading its fragments straight from global memory
// (16 bytes per lane and fragment, UNROLL k-steps in flight), AT token blocks of
// 32 against one feature block.  The KS partial tiles are added through LDS in a
// fixed order.
template <int AT, int KS, int UNROLL>
__global__ __launch_bounds__(64 * KS) void linear_skinny_kernel(
    const half_t *__restrict__ x, const half_t *__restrict__ w, const half_t *__restrict__ bias,
    half_t *__restrict__ y, int T, int M, int N) {
    __shared__ float red[KS][AT][16][64];
    const int lane = threadIdx.x & 63, ks = threadIdx.x >> 6;
    const int l32 = lane & 31, kh = lane >> 5;
    const int m0 = blockIdx.x * 32;
    // this wave's share of the k-steps (16 columns each)
    const int steps = N / 16, per = (steps + KS - 1) / KS;
    const int s_begin = ks * per, s_end = min(s_begin + per, steps);

    const half_t *wp = w + (int64_t)min(m0 + l32, M - 1) * N + 8 * kh;
    const half_t *xp[AT];
#pragma unroll
    for (int a = 0; a < AT; a++) xp[a] = x + (int64_t)min(32 * a + l32, T - 1) * N + 8 * kh;

    float16_t acc[AT];
#pragma unroll
    for (int a = 0; a < AT; a++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[a][v] = 0.f;

    for (int st = s_begin; st < s_end; st += UNROLL) {
        half8_t bf[UNROLL], af[UNROLL][AT];
#pragma unroll
        for (int q = 0; q < UNROLL; q++) {
            const int k = min(st + q, s_end - 1) * 16;     // clamped: the surplus products are skipped below
            bf[q] = *reinterpret_cast<const half8_t *>(wp + k);
#pragma unroll
            for (int a = 0; a < AT; a++) af[q][a] = *reinterpret_cast<const half8_t *>(xp[a] + k);
        }
#pragma unroll
        for (int q = 0; q < UNROLL; q++) {
            if (st + q < s_end) {
#pragma unroll
                for (int a = 0; a < AT; a++)
                    acc[a] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[q][a], bf[q], acc[a], 0, 0, 0);
            }
        }
    }

#pragma unroll
    for (int a = 0; a < AT; a++)
#pragma unroll
        for (int v = 0; v < 16; v++) red[ks][a][v][lane] = acc[a][v];
    __syncthreads();
    // D[token, feature]: lane holds feature l32, tokens 8 * (v / 4) + 4 * kh + v % 4
    for (int item = ks; item < AT * 16; item += KS) {
        const int a = item / 16, v = item % 16;
        float sum = 0.f;
#pragma unroll
        for (int k = 0; k < KS; k++) sum += red[k][a][v][lane];
        const int m = m0 + l32, t = 32 * a + 8 * (v >> 2) + 4 * kh + (v & 3);
        if (m < M && t < T) y[(int64_t)t * M + m] = (half_t)(sum + (bias ? (float)bias[m] : 0.f));
    }
}

// Shapes the tiled kernel does not take (N % 8 != 0 or unaligned buffers).
__global__ __launch_bounds__(256) void linear_generic_kernel(
    const half_t *__restrict__ x, const half_t *__restrict__ w, const half_t *__restrict__ bias,
    half_t *__restrict__ y, int T, int M, int N) {
    // one wave per output element, lanes stride over n
    const int lane = threadIdx.x & 63;
    int64_t o = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int64_t total = (int64_t)T * M;
    const int64_t stride = ((int64_t)gridDim.x * blockDim.x) >> 6;
    for (; o < total; o += stride) {
        const int t = (int)(o / M), m = (int)(o % M);
        float acc = 0.f;
        for (int n = lane; n < N; n += 64)
            acc = __builtin_fmaf((float)x[(int64_t)t * N + n], (float)w[(int64_t)m * N + n], acc);
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
        if (lane == 0) y[o] = (half_t)(acc + (bias ? (float)bias[m] : 0.f));
    }
}

// NS: register sets of pieces in flight.  TAILS: also instantiate the kernel for a contracted range that ends in a partial
// k-step (false: the caller only comes with N % GK == 0).
template <int WT, int WF, int AT, int AF, int GK, int NS = 3, bool TAILS = true>
int launch_tiled(const half_t *x, const half_t *w, const half_t *bias, half_t *y, int T, int M, int N,
                 hipStream_t s) {
    constexpr int BT = WT * AT * 32, BF = WF * AF * 32;
    constexpr size_t lds = (size_t)2 * (BT + BF) * lds_stride(GK) * sizeof(half_t);
    static bs_lds_grant granted[2][BS_MAX_DEVICES];
    int st = bs_allow_lds((const void *)linear_f16_kernel<WT, WF, AT, AF, GK, false, NS>, lds, granted[0]);
    if constexpr (TAILS) {
        if (st == BS_OK) st = bs_allow_lds((const void *)linear_f16_kernel<WT, WF, AT, AF, GK, true, NS>, lds, granted[1]);
    }
    if (st != BS_OK) return st;
    dim3 grid((unsigned)bs_cdiv(M, BF), (unsigned)bs_cdiv(T, BT));
    if (N % GK == 0) {
        linear_f16_kernel<WT, WF, AT, AF, GK, false, NS><<<grid, 64 * WT * WF, lds, s>>>(x, w, bias, y, T, M, N);
    } else {
        if constexpr (TAILS)
            linear_f16_kernel<WT, WF, AT, AF, GK, true, NS><<<grid, 64 * WT * WF, lds, s>>>(x, w, bias, y, T, M, N);
        else
            return BS_ERR_SHAPE;
    }
    return BS_OK;
}

}  // namespace

// Which kernel a dense forward of these dimensions runs: tokens x features per workgroup
// (0 x 0 for the one-wave-per-output kernel), and whether the contracted range ends in a
// partial k-step.
struct LinearTile { int bt, bf, gk; };
static LinearTile linear_tile(int T, int M, int N, bool aligned) {
    if (!(N % 8 == 0 && aligned) || N >= (1 << 23)) return {0, 0, 0};     // (a tile's rows stay within 32-bit byte offsets)
    if (T <= 32 && N % 16 == 0) return {32, 32, 0};                       // linear_skinny_kernel
    if (T <= 128) return M >= 8192 ? LinearTile{128, 64, 64} : LinearTile{128, 32, 128};
    // The largest tile whose grid still covers most of the 256 CUs: 256 x 256 and
    // 128 x 256 (8 waves) move the fewest bytes per flop; 128 x 128 and 64 x 64
    // (4 waves, two workgroups per CU) keep a small problem spread over the chip.
    const auto wgs = [&](int bt, int bf) { return bs_cdiv(T, bt) * bs_cdiv(M, bf); };
    return wgs(256, 256) >= 160 ? LinearTile{256, 256, N % 64 == 0 ? 64 : 32} :
           wgs(128, 256) >= 160 ? LinearTile{128, 256, 64} :
           wgs(128, 128) >= 160 ? LinearTile{128, 128, 64} : LinearTile{64, 64, 128};
}

int bs_launch_linear_f16(const half_t *x, const half_t *w, const half_t *bias, half_t *y,
                         int T, int M, int N, hipStream_t s) {
    const LinearTile tile = linear_tile(T, M, N, bs_aligned(x, 16) && bs_aligned(w, 16));
    int st = BS_OK;
    if (tile.bt == 0) {
        int64_t blocks = bs_cdiv((int64_t)T * M, 4);
        if (blocks > 256 * 64) blocks = 256 * 64;
        linear_generic_kernel<<<(int)blocks, 256, 0, s>>>(x, w, bias, y, T, M, N);
    } else if (tile.gk == 0) {
        linear_skinny_kernel<1, 8, 8><<<(int)bs_cdiv(M, 32), 512, 0, s>>>(x, w, bias, y, T, M, N);
    } else if (tile.bt == 128 && tile.bf == 64) {
        st = launch_tiled<2, 2, 2, 1, 64>(x, w, bias, y, T, M, N, s);
    } else if (tile.bt == 128 && tile.bf == 32) {
        st = launch_tiled<4, 1, 1, 1, 128>(x, w, bias, y, T, M, N, s);
    } else if (tile.bt == 256 && tile.gk == 64) {
        st = launch_tiled<2, 4, 4, 2, 64, 2, false>(x, w, bias, y, T, M, N, s);
    } else if (tile.bt == 256) {
        st = launch_tiled<2, 4, 4, 2, 32>(x, w, bias, y, T, M, N, s);
    } else if (tile.bf == 256) {
        st = launch_tiled<2, 4, 2, 2, 64, 4>(x, w, bias, y, T, M, N, s);
    } else if (tile.bf == 128) {
        st = launch_tiled<2, 2, 2, 2, 64, 4>(x, w, bias, y, T, M, N, s);
    } else {
        st = launch_tiled<2, 2, 1, 1, 128, 4>(x, w, bias, y, T, M, N, s);
    }
    if (st != BS_OK) return st;
    BS_LAUNCH_CHECK();
    return BS_OK;
}

extern "C" int bs_linear_plan(int T, int M, int N, int *tile_tokens, int *tile_features, int *k_step, int *k_tail) {
    if (!tile_tokens || !tile_features || !k_step || !k_tail) return BS_ERR_NULL;
    if (T <= 0 || M <= 0 || N <= 0) return BS_ERR_SHAPE;
    const LinearTile t = linear_tile(T, M, N, true);
    *tile_tokens = t.bt;
    *tile_features = t.bf;
    *k_step = t.gk;
    *k_tail = t.gk > 0 && N % t.gk != 0;
    return BS_OK;
}

extern "C" int bs_linear_f16(const void *x, const void *w, const void *bias, void *y,
                             int T, int M, int N, void *stream) {
    if (T < 0 || M <= 0 || N <= 0) return BS_ERR_SHAPE;
    if (T == 0) return BS_OK;
    if (!x || !w || !y) return BS_ERR_NULL;
    if (!bs_aligned(x, 2) || !bs_aligned(w, 2) || !bs_aligned(y, 2) || !bs_aligned(bias, 2))
        return BS_ERR_ALIGN;
    return bs_launch_linear_f16((const half_t *)x, (const half_t *)w, (const half_t *)bias,
                                (half_t *)y, T, M, N, (hipStream_t)stream);
}

// Dense fp16 contraction y[T, M] = x[T, N] @ w[M, N]^T (+ bias) on gfx950 MFMA.
//
// Both operands are contiguous along the contracted index N, which is what
// v_mfma_f32_32x32x16_f16 wants: a lane supplies eight consecutive k of one
// row (A = tokens) or one column (B = features), i.e. one 16-byte read per
// fragment.
//
// More than 128 tokens: linear_f16_kernel, 2 x 2 waves of 2 x 2 MFMA tiles
// (128 tokens x 128 features per workgroup), k-steps of 64 columns through LDS;
// rows are padded by 8 halves so that the eight lanes served per LDS cycle hit
// disjoint banks.  Global loads for step s+1 are issued before the MFMAs of
// step s (register staging, two LDS buffers, one barrier per step).  Larger
// per-wave tiles (4 x 2, 2 x 4) and 32-column steps measured slower: with one
// step of look-ahead the kernel is bound by load latency, not by LDS traffic.
// 33..128 tokens use narrower workgroups of the same kernel (more workgroups for
// the few token rows); up to 32 tokens: linear_skinny_kernel (below).
#include "common.h"

namespace {


template <int WT, int WF, int AT, int AF, int GK>
__global__ __launch_bounds__(64 * WT * WF) void linear_f16_kernel(
    const half_t *__restrict__ x, const half_t *__restrict__ w, const half_t *__restrict__ bias,
    half_t *__restrict__ y, int T, int M, int N) {
    constexpr int THREADS = 64 * WT * WF;
    constexpr int BT = WT * AT * 32, BF = WF * AF * 32;      // workgroup tile: tokens x features
    constexpr int ROWS = BT + BF;                            // LDS rows per buffer (x rows, then w rows)
    constexpr int PPR = GK / 8;                              // 16-byte pieces per row and k-step
    constexpr int LSTRIDE = GK + 8;                          // halves per LDS row (padded)
    constexpr int PIECES = ROWS * PPR;                       // 16-byte pieces per k-step
    constexpr int PER_THREAD = (PIECES + THREADS - 1) / THREADS;
    extern __shared__ __attribute__((aligned(16))) half_t lds_raw[];
    half_t (*lds)[ROWS * (GK + 8)] = reinterpret_cast<half_t (*)[ROWS * (GK + 8)]>(lds_raw);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int t0 = blockIdx.y * BT, m0 = blockIdx.x * BF;
    const int wt = (wave / WF) * (AT * 32), wf = (wave % WF) * (AF * 32);
    const int l32 = lane & 31, kh = lane >> 5;

    // loader role: piece p = tid + THREADS * j -> LDS row p / PPR, 16-byte piece p % PPR
    const half_t *src[PER_THREAD];
    int dst[PER_THREAD];
    bool live[PER_THREAD];
#pragma unroll
    for (int j = 0; j < PER_THREAD; j++) {
        const int p = tid + THREADS * j, row = p / PPR, piece = p % PPR;
        live[j] = p < PIECES;
        const int r = live[j] ? row : 0;
        src[j] = (r < BT ? x + (int64_t)min(t0 + r, T - 1) * N : w + (int64_t)min(m0 + r - BT, M - 1) * N) + 8 * piece;
        dst[j] = r * LSTRIDE + 8 * piece;
    }

    float16_t acc[AT][AF];
#pragma unroll
    for (int a = 0; a < AT; a++)
#pragma unroll
        for (int b = 0; b < AF; b++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[a][b][v] = 0.f;

    const int steps = (N + GK - 1) / GK;
    uint4_t stage[PER_THREAD];
    auto fetch = [&](int step) {
#pragma unroll
        for (int j = 0; j < PER_THREAD; j++) {
            const int piece = (tid + THREADS * j) % PPR;
            const bool in = live[j] && step * GK + 8 * piece < N;     // N % 8 == 0: a piece is all in or all out
            stage[j] = in ? *reinterpret_cast<const uint4_t *>(src[j] + step * GK) : (uint4_t){0, 0, 0, 0};
        }
    };
    auto stash = [&](int buf) {
#pragma unroll
        for (int j = 0; j < PER_THREAD; j++)
            if (live[j]) *reinterpret_cast<uint4_t *>(&lds[buf][dst[j]]) = stage[j];
    };

    fetch(0);
    stash(0);
    __syncthreads();
    for (int step = 0; step < steps; step++) {
        const int buf = step & 1;
        if (step + 1 < steps) fetch(step + 1);
        const half_t *xs = &lds[buf][0], *ws = &lds[buf][BT * LSTRIDE];
#pragma unroll
        for (int kk = 0; kk < GK / 16; kk++) {
            half8_t a[AT], b[AF];
#pragma unroll
            for (int j = 0; j < AT; j++)
                a[j] = *reinterpret_cast<const half8_t *>(xs + (wt + 32 * j + l32) * LSTRIDE + 16 * kk + 8 * kh);
#pragma unroll
            for (int j = 0; j < AF; j++)
                b[j] = *reinterpret_cast<const half8_t *>(ws + (wf + 32 * j + l32) * LSTRIDE + 16 * kk + 8 * kh);
#pragma unroll
            for (int ai = 0; ai < AT; ai++)
#pragma unroll
                for (int bi = 0; bi < AF; bi++)
                    acc[ai][bi] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[ai], b[bi], acc[ai][bi], 0, 0, 0);
        }
        if (step + 1 < steps) stash(buf ^ 1);
        __syncthreads();
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

template <int WT, int WF, int AT, int AF, int GK>
int launch_tiled(const half_t *x, const half_t *w, const half_t *bias, half_t *y, int T, int M, int N,
                 hipStream_t s) {
    constexpr int BT = WT * AT * 32, BF = WF * AF * 32;
    constexpr size_t lds = (size_t)2 * (BT + BF) * (GK + 8) * sizeof(half_t);
    static bool raised = false;
    if (lds > 64 * 1024 && !raised) {
        BS_HIP_TRY(hipFuncSetAttribute((const void *)linear_f16_kernel<WT, WF, AT, AF, GK>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        raised = true;
    }
    dim3 grid((unsigned)bs_cdiv(M, BF), (unsigned)bs_cdiv(T, BT));
    linear_f16_kernel<WT, WF, AT, AF, GK><<<grid, 64 * WT * WF, lds, s>>>(x, w, bias, y, T, M, N);
    return BS_OK;
}

}  // namespace

int bs_launch_linear_f16(const half_t *x, const half_t *w, const half_t *bias, half_t *y,
                         int T, int M, int N, hipStream_t s) {
    if (N % 8 == 0 && bs_aligned(x, 16) && bs_aligned(w, 16)) {
        int st = BS_OK;
        if (T <= 32 && N % 16 == 0) {
            linear_skinny_kernel<1, 8, 8><<<(int)bs_cdiv(M, 32), 512, 0, s>>>(x, w, bias, y, T, M, N);
        } else if (T <= 128) {
            st = M >= 8192 ? launch_tiled<2, 2, 2, 1, 64>(x, w, bias, y, T, M, N, s)
                           : launch_tiled<4, 1, 1, 1, 128>(x, w, bias, y, T, M, N, s);
        } else {
            st = launch_tiled<2, 2, 2, 2, 64>(x, w, bias, y, T, M, N, s);
        }
        if (st != BS_OK) return st;
    } else {
        int64_t blocks = bs_cdiv((int64_t)T * M, 4);
        if (blocks > 256 * 64) blocks = 256 * 64;
        linear_generic_kernel<<<(int)blocks, 256, 0, s>>>(x, w, bias, y, T, M, N);
    }
    BS_LAUNCH_CHECK();
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

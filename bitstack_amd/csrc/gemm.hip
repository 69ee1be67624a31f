// Dense fp16 contraction y[T, M] = x[T, N] @ w[M, N]^T (+ bias) on gfx950 MFMA.
//
// Both operands are contiguous along the contracted index N, which is what
// v_mfma_f32_32x32x16_f16 wants: a lane supplies eight consecutive k of one
// row (A) or one column (B), i.e. one 16-byte read per fragment.
//
// Workgroup = 256 threads = 4 waves, output tile 128 tokens x 128 features,
// each wave a 64 x 64 quadrant (2 x 2 MFMA tiles, 64 fp32 accumulators).
// The k-loop steps 32 columns at a time through LDS; rows are padded to 40
// halves (80 B) so that the eight lanes served per LDS cycle hit disjoint
// banks.  Global loads for step s+1 are issued before the MFMAs of step s.
#include "common.h"

namespace {

constexpr int GT = 128;       // tokens per workgroup
constexpr int GM = 128;       // features per workgroup
constexpr int GK = 32;        // k per step
constexpr int LSTRIDE = 40;   // halves per LDS row

__global__ __launch_bounds__(256) void linear_f16_kernel(
    const half_t *__restrict__ x, const half_t *__restrict__ w, const half_t *__restrict__ bias,
    half_t *__restrict__ y, int T, int M, int N) {
    __shared__ __attribute__((aligned(16))) half_t xs[2][GT * LSTRIDE];
    __shared__ __attribute__((aligned(16))) half_t ws[2][GM * LSTRIDE];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int t0 = blockIdx.y * GT, m0 = blockIdx.x * GM;
    const int wt = (wave >> 1) * 64, wm = (wave & 1) * 64;
    const int l32 = lane & 31, kh = lane >> 5;

    // loader role: 4 pieces of 8 halves per row, 64 rows per pass, 2 passes
    const int lrow = tid >> 2, lpiece = tid & 3;
    const half_t *xg[2], *wg[2];
#pragma unroll
    for (int j = 0; j < 2; j++) {
        xg[j] = x + (int64_t)min(t0 + lrow + 64 * j, T - 1) * N + 8 * lpiece;
        wg[j] = w + (int64_t)min(m0 + lrow + 64 * j, M - 1) * N + 8 * lpiece;
    }

    float16_t acc[2][2];
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
        for (int b = 0; b < 2; b++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[a][b][v] = 0.f;

    const int steps = (N + GK - 1) / GK;
    uint4_t xr[2], wr[2];
    auto fetch = [&](int step) {
        const int k = step * GK + 8 * lpiece;
        const bool in = k < N;           // N % 8 == 0: a piece is all in or all out
#pragma unroll
        for (int j = 0; j < 2; j++) {
            xr[j] = in ? *reinterpret_cast<const uint4_t *>(xg[j] + step * GK) : (uint4_t){0, 0, 0, 0};
            wr[j] = in ? *reinterpret_cast<const uint4_t *>(wg[j] + step * GK) : (uint4_t){0, 0, 0, 0};
        }
    };
    auto stash = [&](int buf) {
#pragma unroll
        for (int j = 0; j < 2; j++) {
            *reinterpret_cast<uint4_t *>(&xs[buf][(lrow + 64 * j) * LSTRIDE + 8 * lpiece]) = xr[j];
            *reinterpret_cast<uint4_t *>(&ws[buf][(lrow + 64 * j) * LSTRIDE + 8 * lpiece]) = wr[j];
        }
    };

    fetch(0);
    stash(0);
    __syncthreads();
    for (int step = 0; step < steps; step++) {
        const int buf = step & 1;
        if (step + 1 < steps) fetch(step + 1);
#pragma unroll
        for (int kk = 0; kk < 2; kk++) {
            half8_t a[2], b[2];
#pragma unroll
            for (int j = 0; j < 2; j++) {
                a[j] = *reinterpret_cast<const half8_t *>(&xs[buf][(wt + 32 * j + l32) * LSTRIDE + 16 * kk + 8 * kh]);
                b[j] = *reinterpret_cast<const half8_t *>(&ws[buf][(wm + 32 * j + l32) * LSTRIDE + 16 * kk + 8 * kh]);
            }
#pragma unroll
            for (int ai = 0; ai < 2; ai++)
#pragma unroll
                for (int bi = 0; bi < 2; bi++)
                    acc[ai][bi] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[ai], b[bi], acc[ai][bi], 0, 0, 0);
        }
        if (step + 1 < steps) stash(buf ^ 1);
        __syncthreads();
    }

    // D[token, feature]: lane holds feature l32, tokens 8 * (v / 4) + 4 * kh + v % 4
#pragma unroll
    for (int bi = 0; bi < 2; bi++) {
        const int m = m0 + wm + 32 * bi + l32;
        if (m >= M) continue;
        const float bv = bias ? (float)bias[m] : 0.f;
#pragma unroll
        for (int ai = 0; ai < 2; ai++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int t = t0 + wt + 32 * ai + 8 * (v >> 2) + 4 * kh + (v & 3);
                if (t < T) y[(int64_t)t * M + m] = (half_t)(acc[ai][bi][v] + bv);
            }
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

}  // namespace

int bs_launch_linear_f16(const half_t *x, const half_t *w, const half_t *bias, half_t *y,
                         int T, int M, int N, hipStream_t s) {
    if (N % 8 == 0 && bs_aligned(x, 16) && bs_aligned(w, 16)) {
        dim3 grid((unsigned)bs_cdiv(M, GM), (unsigned)bs_cdiv(T, GT));
        linear_f16_kernel<<<grid, 256, 0, s>>>(x, w, bias, y, T, M, N);
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

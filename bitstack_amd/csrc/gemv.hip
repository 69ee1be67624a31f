// Packed-sign GEMV for decode (1..8 tokens) on gfx950.
//
//   y[t, m] = sum_i sum_r u_i[m, r] * ( sum_n s_i[m, n] * vt_i[r, n] * x[t, n] )
//
// The inner sum is a matrix product  Z_i,t (16 x N)  x  S_i^T (N x rows)  with
// Z_i,t[r, n] = vt_i[r, n] * x[t, n], so it runs on v_mfma_f32_16x16x32_f16:
// A = a 16 x 32 patch of Z (fp16), B = 32 signs of 16 rows as fp16 +-1,
// D[r, m] accumulated in fp32 over the whole slice of n a workgroup owns.  A
// lane then holds four ranks of ONE row, multiplies them by u_i[m, 4g..4g+3],
// and two cross-lane adds finish the row.
//
// Work split: workgroup = (row tile of 64*R rows, block i, group of 512-column
// chunks).  The four waves take 16*R rows each and share Z through LDS; every
// lane reads its 16 bytes of signs (128 columns of one row) with one 128-bit
// load per chunk and row tile.  Partial row sums go to a scratch array
// [I * groups, T, M] (fp32) and a second small kernel adds them in a fixed
// order, adds the bias and rounds to fp16 - deterministic, no atomics.
//
// Sign decode.  A lane's 16 bytes are four little-endian words w0..w3.  MFMA
// number c (0..15) of a chunk takes bits c and c+16 of each word: after
// `w << (15 - c)` they sit in the two fp16 sign positions, and one
// v_and_or_b32 with 0x80008000 / 0x3C003C00 yields the pair (+-1, +-1).  A set
// bit thus decodes to -1 whereas the storage format says +1, so Z is produced
// negated.  Which column a given MFMA k-slot sees follows from this bit
// choice, and Z is laid out in LDS in exactly that order:
//   slot s = 2p + h of lane group g in MFMA c  <->  column
//   128 g + 32 p + 16 h + 8 (c / 8) + 7 - c % 8   of the chunk.
#include "common.h"

namespace {

constexpr int CH = 512;   // columns per chunk: 4 lane groups x 16 bytes of signs

// LDS image of Z for one chunk: [t][c (16)][g (4)][r (16)][slot (8)] halves.
__device__ inline int z_index(int t, int c, int g, int r) { return (((t * 16 + c) * 4 + g) * 16 + r) * 8; }

template <int T, int R>
__global__ __launch_bounds__(256) void gemv_kernel(
    const uint8_t *__restrict__ packed, const half_t *__restrict__ u, const half_t *__restrict__ vt,
    const half_t *__restrict__ x, float *__restrict__ part,
    int I, int M, int N, int K, int row_tiles, int groups, int chunks_per_group, int n_chunks) {
    extern __shared__ __attribute__((aligned(16))) half_t zl[];   // T * 16 KB

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lm = lane & 15, g = lane >> 4;
    const int rt = blockIdx.x % row_tiles;
    const int task = blockIdx.x / row_tiles;          // = i * groups + cg
    const int i = task / groups, cg = task % groups;
    const int c_begin = cg * chunks_per_group;
    const int c_end = min(c_begin + chunks_per_group, n_chunks);

    const int64_t row_bytes = N >> 3;
    const uint8_t *qi = packed + (int64_t)i * M * row_bytes;
    const half_t *vti = vt + (int64_t)i * K * N;

    int rowbase[R];
    const uint8_t *qrow[R];
#pragma unroll
    for (int jr = 0; jr < R; jr++) {
        rowbase[jr] = rt * (64 * R) + (wave * R + jr) * 16;
        qrow[jr] = qi + (int64_t)min(rowbase[jr] + lm, M - 1) * row_bytes + 16 * g;
    }

    float4_t acc[R][T];
#pragma unroll
    for (int jr = 0; jr < R; jr++)
#pragma unroll
        for (int t = 0; t < T; t++) acc[jr][t] = (float4_t){0.f, 0.f, 0.f, 0.f};

    for (int c = c_begin; c < c_end; c++) {
        const int cb = c * CH;
        // signs first: their latency hides behind the production of Z
        uint4_t sw[R];
#pragma unroll
        for (int jr = 0; jr < R; jr++) sw[jr] = *reinterpret_cast<const uint4_t *>(qrow[jr] + (cb >> 3));

        if (c != c_begin) __syncthreads();   // everyone is done reading the previous Z
        for (int item = tid; item < T * 128; item += 256) {
            const int r = item & 15, pg = (item >> 4) & 3, jb = (item >> 6) & 1, t = item >> 7;
            half8_t z[8];
#pragma unroll
            for (int s = 0; s < 8; s++) {
                const int noff = cb + 128 * pg + 32 * (s >> 1) + 16 * (s & 1) + 8 * jb;
                half8_t xv = *reinterpret_cast<const half8_t *>(x + (int64_t)t * N + noff);
                half8_t vv = {0, 0, 0, 0, 0, 0, 0, 0};
                if (r < K) vv = *reinterpret_cast<const half8_t *>(vti + (int64_t)r * N + noff);
                z[s] = -(vv * xv);
            }
#pragma unroll
            for (int e = 0; e < 8; e++) {
                half8_t o = {z[0][e], z[1][e], z[2][e], z[3][e], z[4][e], z[5][e], z[6][e], z[7][e]};
                *reinterpret_cast<half8_t *>(&zl[z_index(t, 8 * jb + 7 - e, pg, r)]) = o;
            }
        }
        __syncthreads();

#pragma unroll
        for (int cls = 0; cls < 16; cls++) {
            half8_t zf[T];
#pragma unroll
            for (int t = 0; t < T; t++) zf[t] = *reinterpret_cast<const half8_t *>(&zl[z_index(t, cls, g, lm)]);
#pragma unroll
            for (int jr = 0; jr < R; jr++) {
                uint4_t sb;
#pragma unroll
                for (int p = 0; p < 4; p++) sb[p] = ((sw[jr][p] << (15 - cls)) & 0x80008000u) | 0x3C003C00u;
                const half8_t sf = __builtin_bit_cast(half8_t, sb);
#pragma unroll
                for (int t = 0; t < T; t++)
                    acc[jr][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(zf[t], sf, acc[jr][t], 0, 0, 0);
            }
        }
    }

    // D[r, m]: this lane holds ranks 4g..4g+3 of row rowbase + lm
#pragma unroll
    for (int jr = 0; jr < R; jr++) {
        const int row = rowbase[jr] + lm;
        const half_t *up = u + ((int64_t)i * M + min(row, M - 1)) * K + 4 * g;
        float uf[4];
#pragma unroll
        for (int v = 0; v < 4; v++) uf[v] = (4 * g + v < K) ? (float)up[v] : 0.f;
#pragma unroll
        for (int t = 0; t < T; t++) {
            float val = acc[jr][t][0] * uf[0] + acc[jr][t][1] * uf[1] + acc[jr][t][2] * uf[2] + acc[jr][t][3] * uf[3];
            val += __shfl_xor(val, 16, 64);
            val += __shfl_xor(val, 32, 64);
            if (g == 0 && row < M) part[((int64_t)task * T + t) * M + row] = val;
        }
    }
}

// y[t, m] = fp16( sum_k part[k, t, m] + bias[m] ), k ascending.
__global__ __launch_bounds__(256) void gemv_reduce_kernel(const float *__restrict__ part,
                                                          const half_t *__restrict__ bias,
                                                          half_t *__restrict__ y, int KP, int T, int M) {
    const int64_t total = (int64_t)T * M;
    const int64_t o = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (o >= total) return;
    float acc = 0.f;
    for (int k = 0; k < KP; k++) acc += part[(int64_t)k * total + o];
    if (bias) acc += (float)bias[o % M];
    y[o] = (half_t)acc;
}

struct Plan {
    int R, row_tiles, groups, chunks_per_group, n_chunks;
};

Plan make_plan(int I, int M, int N) {
    Plan p;
    p.n_chunks = N / CH;
    const int64_t want = 768;   // workgroups that keep 256 CUs busy with some slack
    p.R = 1;
    for (int r = 4; r >= 1; r >>= 1) {
        if (bs_cdiv(M, 64 * r) * I * p.n_chunks >= want || r == 1) { p.R = r; break; }
    }
    p.row_tiles = (int)bs_cdiv(M, 64 * p.R);
    // merge chunks into groups while enough workgroups remain
    int cpg = 1;
    while (cpg * 2 <= p.n_chunks && (int64_t)p.row_tiles * I * bs_cdiv(p.n_chunks, cpg * 2) >= want) cpg *= 2;
    p.chunks_per_group = cpg;
    p.groups = (int)bs_cdiv(p.n_chunks, cpg);
    return p;
}

template <int T>
int launch_T(const Plan &p, const uint8_t *packed, const half_t *u, const half_t *vt, const half_t *x,
             float *part, int I, int M, int N, int K, hipStream_t s) {
    const int grid = p.row_tiles * I * p.groups;
    const size_t lds = (size_t)T * 16 * 1024;
#define BS_GEMV_LAUNCH(RR)                                                                        \
    do {                                                                                          \
        if (lds > 48 * 1024)                                                                      \
            BS_HIP_TRY(hipFuncSetAttribute((const void *)gemv_kernel<T, RR>,                       \
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds)); \
        gemv_kernel<T, RR><<<grid, 256, lds, s>>>(packed, u, vt, x, part, I, M, N, K, p.row_tiles, \
                                                  p.groups, p.chunks_per_group, p.n_chunks);      \
    } while (0)
    if (p.R == 4) BS_GEMV_LAUNCH(4);
    else if (p.R == 2) BS_GEMV_LAUNCH(2);
    else BS_GEMV_LAUNCH(1);
#undef BS_GEMV_LAUNCH
    BS_LAUNCH_CHECK();
    return BS_OK;
}

}  // namespace

static bool gemv_shape_ok(int I, int M, int N, int T) {
    return I >= 1 && T >= 1 && T <= 8 && N % CH == 0 && M >= 1;
}

int64_t bs_gemv_workspace_bytes(int I, int M, int N, int K, int T) {
    (void)K;
    if (!gemv_shape_ok(I, M, N, T)) return 0;
    Plan p = make_plan(I, M, N);
    return (int64_t)I * p.groups * T * M * (int64_t)sizeof(float);
}

// Returns BS_ERR_SHAPE when the fast path does not apply (the caller falls
// back to rebuilding the weight); any other status is final.
int bs_launch_gemv(const uint8_t *packed, const half_t *u, const half_t *vt, const half_t *x,
                   const half_t *bias, half_t *y, int I, int M, int N, int K, int T,
                   void *workspace, int64_t workspace_bytes, hipStream_t s) {
    if (!gemv_shape_ok(I, M, N, T)) return BS_ERR_SHAPE;
    if (!bs_aligned(packed, 16) || !bs_aligned(vt, 16) || !bs_aligned(x, 16)) return BS_ERR_SHAPE;
    Plan p = make_plan(I, M, N);
    const int64_t need = (int64_t)I * p.groups * T * M * (int64_t)sizeof(float);
    if (!workspace || workspace_bytes < need) return BS_ERR_WORKSPACE;
    float *part = (float *)workspace;
    int st;
    switch (T) {
        case 1: st = launch_T<1>(p, packed, u, vt, x, part, I, M, N, K, s); break;
        case 2: st = launch_T<2>(p, packed, u, vt, x, part, I, M, N, K, s); break;
        case 3: st = launch_T<3>(p, packed, u, vt, x, part, I, M, N, K, s); break;
        case 4: st = launch_T<4>(p, packed, u, vt, x, part, I, M, N, K, s); break;
        case 5: st = launch_T<5>(p, packed, u, vt, x, part, I, M, N, K, s); break;
        case 6: st = launch_T<6>(p, packed, u, vt, x, part, I, M, N, K, s); break;
        case 7: st = launch_T<7>(p, packed, u, vt, x, part, I, M, N, K, s); break;
        default: st = launch_T<8>(p, packed, u, vt, x, part, I, M, N, K, s); break;
    }
    if (st != BS_OK) return st;
    const int64_t total = (int64_t)T * M;
    gemv_reduce_kernel<<<(int)bs_cdiv(total, 256), 256, 0, s>>>(part, bias, y, I * p.groups, T, M);
    BS_LAUNCH_CHECK();
    return BS_OK;
}

// Types shared by the decode kernels (gemv.hip, gemv_mx.hip): the static partition of
// units over workgroups and the by-value argument block of a grouped launch.
#pragma once

#include "common.h"

// Static partition of U units over G workgroups: the first `rem` get q + 1.
struct Split {
    int q, rem;
    __host__ __device__ int start(int w) const { return w * q + (w < rem ? w : rem); }
    __host__ __device__ int owner(int unit) const {
        const int big = rem * (q + 1);
        return unit < big ? unit / (q + 1) : rem + (unit - big) / q;
    }
};

// Up to GEMV_MAX_GROUP matrices that share x (and so N and K) run in one launch:
// the grid is cut into one run of workgroups per matrix, each with its own static
// partition, partial-sum area and row count.
constexpr int GEMV_MAX_GROUP = 4;
constexpr int GEMV_WIDE_MIN_UNITS = 1024;   // 1024-row units from which one token runs on 16-wave workgroups
constexpr int GEMV_PAIR_MIN_UNITS = 4;      // units per workgroup from which workgroups are paired
struct GemvMat {
    const uint8_t *packed;
    const half_t *u, *vt;
    float *part;
    int M, row_tiles, kmax, first_wg;
    Split sp;
    // 1: workgroups 2p and 2p + 1 share one range of (block, row tile, chunk PAIR) units and
    // take the even / the odd 512-column chunk of every pair.  The two 64-byte halves of a
    // 128-byte line of sign bytes are then requested at about the same time by neighbours on
    // one XCD (the second request hits L2) instead of one unit apart by the same workgroup,
    // by when the line has often been evicted and comes from HBM again.
    int pair;
};
struct GemvGroup {
    GemvMat m[GEMV_MAX_GROUP];
    int n;
};

// One- and two-token decode on the block-scaled fp4 x fp6 MFMA (gemv_mx.hip).  Same unit order, partition,
// partial layout and flush as gemv_kernel, but a unit spans MX_UNIT_COLS / T columns; rows per
// workgroup = 8 waves x R x 16.
constexpr int MX_UNIT_COLS = 1024;
bool bs_gemv_mx_takes(int N, int K, int R, int T);
int bs_launch_gemv_mx(int R, int T, int grid, const GemvGroup &grp, const half_t *x, int N, int K, int n_units, hipStream_t s);

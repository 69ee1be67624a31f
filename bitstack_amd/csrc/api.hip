// C ABI glue: argument validation, path selection, status strings.
#include "common.h"

extern "C" int bs_version(void) { return BS_VERSION_NUMBER; }

extern "C" const char *bs_error_string(int status) {
    switch (status) {
        case BS_OK: return "ok";
        case BS_ERR_NULL: return "a required pointer is NULL";
        case BS_ERR_SHAPE: return "non-positive or unsupported dimension";
        case BS_ERR_RANK: return "rank K must be in 1..16";
        case BS_ERR_ALIGN: return "pointer is not aligned as the entry point requires";
        case BS_ERR_WORKSPACE: return "workspace missing, misaligned or too small";
        case BS_ERR_NO_DEVICE: return "no usable HIP device";
        default: break;
    }
    if (status <= BS_ERR_HIP_BASE) return hipGetErrorString((hipError_t)(BS_ERR_HIP_BASE - status));
    return "unknown status";
}

static int forward_dims(int I, int M, int N, int K, int T) {
    if (I < 0 || M <= 0 || N <= 0 || T < 0) return BS_ERR_SHAPE;
    if (N % 8 != 0) return BS_ERR_SHAPE;
    if (K < 1 || K > 16) return BS_ERR_RANK;
    return BS_OK;
}

static int64_t round_up(int64_t v, int64_t a) { return (v + a - 1) / a * a; }

extern "C" int64_t bs_workspace_bytes(int I, int M, int N, int K, int T) {
    int st = forward_dims(I, M, N, K, T);
    if (st != BS_OK) return st;
    if (T == 0) return 0;
    int64_t gemv = bs_gemv_workspace_bytes(I, M, N, K, T);
    if (gemv > 0) return round_up(gemv, 256);
    return round_up((int64_t)M * N * 2, 256);
}

extern "C" int bs_decode_plan(int I, int M, int N, int K, int T, int *waves, int *row_tiles_per_wave,
                              int *workgroups, int *partials_per_row) {
    if (!waves || !row_tiles_per_wave || !workgroups || !partials_per_row) return BS_ERR_NULL;
    int st = forward_dims(I, M, N, K, T);
    if (st != BS_OK) return st;
    bs_gemv_plan_info(I, M, N, T, waves, row_tiles_per_wave, workgroups, partials_per_row);
    return BS_OK;
}

extern "C" int bs_forward(const uint8_t *packed, const void *u, const void *vt, const void *x,
                          const void *bias, void *y, int I, int M, int N, int K, int T,
                          void *workspace, int64_t workspace_bytes, void *stream) {
    int st = forward_dims(I, M, N, K, T);
    if (st != BS_OK) return st;
    if (T == 0) return BS_OK;
    if (!x || !y || (I > 0 && (!packed || !u || !vt))) return BS_ERR_NULL;
    if (!bs_aligned(packed, 16) || !bs_aligned(vt, 16) || !bs_aligned(x, 16) || !bs_aligned(u, 8) ||
        !bs_aligned(y, 2) || !bs_aligned(bias, 2))
        return BS_ERR_ALIGN;
    const int64_t need = bs_workspace_bytes(I, M, N, K, T);
    if (need > 0 && (!workspace || workspace_bytes < need || !bs_aligned(workspace, 256)))
        return BS_ERR_WORKSPACE;
    hipStream_t s = (hipStream_t)stream;

    if (bs_gemv_workspace_bytes(I, M, N, K, T) > 0) {
        st = bs_launch_gemv(packed, (const half_t *)u, (const half_t *)vt, (const half_t *)x,
                            (const half_t *)bias, (half_t *)y, I, M, N, K, T, workspace,
                            workspace_bytes, s);
        return st;
    }
    half_t *w = (half_t *)workspace;
    st = bs_launch_reconstruct_packed(packed, (const half_t *)u, (const half_t *)vt, w, I, M, N, K, s);
    if (st != BS_OK) return st;
    return bs_launch_linear_f16((const half_t *)x, w, (const half_t *)bias, (half_t *)y, T, M, N, s);
}

// C ABI glue: argument validation, path selection, status strings.
#include "common.h"

#include <mutex>

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
        case BS_ERR_LIBRARY: return "the vendor GEMM library failed after it had accepted the call";
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

// Which kernel multiplies the rebuilt weight: this library's linear_f16_kernel unless the calling thread has asked
// for hipBLASLt with bs_set_dense_kernel(BS_DENSE_LIBRARY) (a comparator for tests and benchmarks: what the
// reference's F.linear runs on ROCm).  The setting belongs to the thread that made it, so a size query and the
// forward that follows it on the same thread always agree, whatever other threads do.
static thread_local int g_dense_kernel = 0;

static bool dense_wants_library(int M, int N) {
    return g_dense_kernel == BS_DENSE_LIBRARY && M % 8 == 0 && N % 8 == 0;
}

// Which kernel runs a forward of 49 tokens or more: by shape (0), or pinned for tests and benchmarks.  Per thread.
static thread_local int g_prefill_kernel = 0;
int bs_prefill_mode() { return g_prefill_kernel; }

extern "C" int bs_set_prefill_kernel(int mode) {
    if (mode < 0 || mode > 3) return BS_ERR_SHAPE;
    g_prefill_kernel = mode;
    return BS_OK;
}

extern "C" int bs_set_dense_kernel(int mode) {
    if (mode < 0 || mode > 2) return BS_ERR_SHAPE;
    g_dense_kernel = mode;
    return BS_OK;
}

// `library_ok`: the dense product may run on hipBLASLt (and then needs its scratch behind the weight)
static int64_t workspace_need(int I, int M, int N, int K, int T, bool library_ok) {
    int st = forward_dims(I, M, N, K, T);
    if (st != BS_OK) return st;
    if (T == 0) return 0;
    int64_t gemv = bs_gemv_workspace_bytes(I, M, N, K, T);
    if (gemv > 0) return round_up(gemv, 256);
    // the rebuilt weight, then the library GEMM's own scratch where that is the kernel
    return round_up((int64_t)M * N * 2, 256) + (library_ok && dense_wants_library(M, N) ? BS_DENSE_LIBRARY_WORKSPACE : 0);
}

extern "C" int64_t bs_workspace_bytes(int I, int M, int N, int K, int T) { return workspace_need(I, M, N, K, T, true); }

extern "C" int bs_decode_plan(int I, int M, int N, int K, int T, int *waves, int *row_tiles_per_wave,
                              int *workgroups, int *partials_per_row) {
    if (!waves || !row_tiles_per_wave || !workgroups || !partials_per_row) return BS_ERR_NULL;
    int st = forward_dims(I, M, N, K, T);
    if (st != BS_OK) return st;
    bs_gemv_plan_info(I, M, N, K, T, waves, row_tiles_per_wave, workgroups, partials_per_row);
    return BS_OK;
}

extern "C" int bs_decode_kernel(int I, int M, int N, int K, int T) {
    int st = forward_dims(I, M, N, K, T);
    if (st != BS_OK) return st;
    return bs_gemv_plan_kernel(I, M, N, K, T);
}

extern "C" int bs_set_decode_kernel(int mode) { return bs_gemv_set_kernel(mode); }

extern "C" int bs_forward_path(int I, int M, int N, int K, int T) {
    int st = forward_dims(I, M, N, K, T);
    if (st != BS_OK) return st;
    if (T == 0 || I == 0) return BS_PATH_REBUILD;      // (no blocks: the weight is zero; the forward still goes through the dense path)
    return bs_gemv_forward_path(I, M, N, K, T);
}

static int forward_impl(const uint8_t *packed, const void *u, const void *vt, const void *x,
                        const void *bias, void *y, int I, int M, int N, int K, int T,
                        void *workspace, int64_t workspace_bytes, void *stream, bool library_ok) {
    int st = forward_dims(I, M, N, K, T);
    if (st != BS_OK) return st;
    if (T == 0) return BS_OK;
    if (!x || !y || (I > 0 && (!packed || !u || !vt))) return BS_ERR_NULL;
    if (!bs_aligned(packed, 16) || !bs_aligned(vt, 16) || !bs_aligned(x, 16) || !bs_aligned(u, 8) ||
        !bs_aligned(y, 2) || !bs_aligned(bias, 2))
        return BS_ERR_ALIGN;
    const int64_t need = workspace_need(I, M, N, K, T, library_ok);
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
    if (library_ok && dense_wants_library(M, N)) {
        st = bs_launch_linear_library((const half_t *)x, w, (const half_t *)bias, (half_t *)y, T, M, N,
                                      (char *)workspace + round_up((int64_t)M * N * 2, 256), s);
        if (st != BS_ERR_SHAPE) return st;      // enqueued, or failed for good; BS_ERR_SHAPE: declined before anything was enqueued
    }
    return bs_launch_linear_f16((const half_t *)x, w, (const half_t *)bias, (half_t *)y, T, M, N, s);
}

extern "C" int bs_forward(const uint8_t *packed, const void *u, const void *vt, const void *x,
                          const void *bias, void *y, int I, int M, int N, int K, int T,
                          void *workspace, int64_t workspace_bytes, void *stream) {
    return forward_impl(packed, u, vt, x, bias, y, I, M, N, K, T, workspace, workspace_bytes, stream, true);
}

// ---- the forward for callers that cannot allocate ------------------------------------
// The scratch of the decode and strip kernels (partial row sums) lives in a file-scope device
// array instead of a caller-owned workspace.  Every GPU the library runs on holds its own copy
// of the array at its own address until the process ends; `scratch` itself is only the
// host-side handle of the symbol, so the address is looked up once per device (with that
// device current) and only the looked-up pointer is ever handed to a kernel.
static __device__ __align__(256) unsigned char scratch[BS_STATIC_SCRATCH_BYTES];
static void *g_scratch_ptr[BS_MAX_DEVICES];
static std::mutex g_scratch_mutex;

static int static_scratch(void **out) {
    int dev = -1;
    BS_HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= BS_MAX_DEVICES) return BS_ERR_NO_DEVICE;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        BS_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p) return BS_ERR_NO_DEVICE;
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return BS_OK;
}

extern "C" int bs_forward_static(const uint8_t *packed, const void *u, const void *vt, const void *x,
                                 const void *bias, void *y, int I, int M, int N, int K, int T, void *stream) {
    int st = forward_dims(I, M, N, K, T);
    if (st != BS_OK) return st;
    if (T == 0) return BS_OK;
    // sizes first: a call that would not fit is refused before any device is touched.  The dense product
    // always runs this library's own kernel here, whatever bs_set_dense_kernel says: the vendor GEMM wants
    // 64 MiB of scratch of its own, and setting it up allocates.
    const int64_t need = workspace_need(I, M, N, K, T, false);
    if (need < 0) return (int)need;
    if (need > (int64_t)BS_STATIC_SCRATCH_BYTES) return BS_ERR_WORKSPACE;
    void *ws = nullptr;
    st = static_scratch(&ws);
    if (st != BS_OK) return st;
    // nothing in the scratch has to start at zero: every partial sum a call reads it has written before
    return forward_impl(packed, u, vt, x, bias, y, I, M, N, K, T, ws, (int64_t)BS_STATIC_SCRATCH_BYTES, stream, false);
}

// ---- grouped decode forward ---------------------------------------------------
static int group_dims(const bs_matrix *mats, int n, int N, int K, int T) {
    if (!mats) return BS_ERR_NULL;
    if (n < 1 || n > BS_MAX_GROUP) return BS_ERR_SHAPE;
    for (int j = 0; j < n; j++) {
        int st = forward_dims(mats[j].I, mats[j].M, N, K, T);
        if (st != BS_OK) return st;
        if (mats[j].I < 1) return BS_ERR_SHAPE;
    }
    if (T < 1 || T > 48) return BS_ERR_SHAPE;
    return BS_OK;
}

extern "C" int64_t bs_forward_group_workspace_bytes(const bs_matrix *mats, int n, int N, int K, int T) {
    int st = group_dims(mats, n, N, K, T);
    if (st != BS_OK) return st;
    int I[BS_MAX_GROUP], M[BS_MAX_GROUP];
    for (int j = 0; j < n; j++) { I[j] = mats[j].I; M[j] = mats[j].M; }
    const int64_t b = bs_gemv_group_workspace_bytes(I, M, n, N, K, T);
    return b > 0 ? round_up(b, 256) : (int64_t)BS_ERR_SHAPE;
}

static int forward_group(const bs_matrix *mats, int n, int N, int K, const void *x, int T,
                         int epilogue, const void *residual, void *y, int input_rms, float eps,
                         void *workspace, int64_t workspace_bytes, void *stream) {
    int st = group_dims(mats, n, N, K, T);
    if (st != BS_OK) return st;
    if (epilogue != BS_EPI_NONE && epilogue != BS_EPI_RESIDUAL && epilogue != BS_EPI_SWIGLU) return BS_ERR_SHAPE;
    if (!x || !y || (epilogue == BS_EPI_RESIDUAL && !residual)) return BS_ERR_NULL;
    const uint8_t *packed[BS_MAX_GROUP];
    const half_t *u[BS_MAX_GROUP], *vt[BS_MAX_GROUP], *bias[BS_MAX_GROUP];
    int I[BS_MAX_GROUP], M[BS_MAX_GROUP];
    for (int j = 0; j < n; j++) {
        if (!mats[j].packed || !mats[j].u || !mats[j].vt) return BS_ERR_NULL;
        if (!bs_aligned(mats[j].packed, 16) || !bs_aligned(mats[j].vt, 16) || !bs_aligned(mats[j].u, 8) ||
            !bs_aligned(mats[j].bias, 2))
            return BS_ERR_ALIGN;
        packed[j] = mats[j].packed;
        u[j] = (const half_t *)mats[j].u;
        vt[j] = (const half_t *)mats[j].vt;
        bias[j] = (const half_t *)mats[j].bias;
        I[j] = mats[j].I;
        M[j] = mats[j].M;
    }
    if (!bs_aligned(x, 16) || !bs_aligned(y, 2) || !bs_aligned(residual, 2)) return BS_ERR_ALIGN;
    const int64_t need = bs_forward_group_workspace_bytes(mats, n, N, K, T);
    if (need < 0) return (int)need;
    if (!workspace || workspace_bytes < need || !bs_aligned(workspace, 256)) return BS_ERR_WORKSPACE;
    return bs_launch_gemv_group(n, packed, u, vt, bias, I, M, N, K, (const half_t *)x, T, epilogue,
                                (const half_t *)residual, (half_t *)y, input_rms, eps, workspace, workspace_bytes,
                                (hipStream_t)stream);
}

extern "C" int bs_forward_group(const bs_matrix *mats, int n, int N, int K, const void *x, int T,
                                int epilogue, const void *residual, void *y,
                                void *workspace, int64_t workspace_bytes, void *stream) {
    return forward_group(mats, n, N, K, x, T, epilogue, residual, y, 0, 0.f, workspace, workspace_bytes, stream);
}

extern "C" int bs_forward_group_rms(const bs_matrix *mats, int n, int N, int K, const void *x, int T, float eps,
                                    int epilogue, const void *residual, void *y,
                                    void *workspace, int64_t workspace_bytes, void *stream) {
    if (!(eps >= 0.f)) return BS_ERR_SHAPE;
    return forward_group(mats, n, N, K, x, T, epilogue, residual, y, 1, eps, workspace, workspace_bytes, stream);
}

extern "C" int bs_rmsnorm_f16(const void *x, const void *weight, void *y, int T, int H, float eps, void *stream) {
    if (T < 0 || H <= 0 || H % 8 != 0 || H > 16384) return BS_ERR_SHAPE;
    if (T == 0) return BS_OK;
    if (!x || !weight || !y) return BS_ERR_NULL;
    if (!bs_aligned(x, 16) || !bs_aligned(weight, 16) || !bs_aligned(y, 16)) return BS_ERR_ALIGN;
    return bs_launch_rmsnorm((const half_t *)x, (const half_t *)weight, (half_t *)y, T, H, eps, (hipStream_t)stream);
}

extern "C" int bs_attention_decode_f16(const void *qkv, void *kcache, void *vcache, const void *cos, const void *sin,
                                       const int64_t *pos, void *out, int B, int heads, int kv_heads, int head_dim,
                                       int max_len, void *stream) {
    if (B < 0 || heads <= 0 || kv_heads <= 0 || heads % kv_heads != 0 || head_dim != 128 || max_len < 1 ||
        max_len > 8192)
        return BS_ERR_SHAPE;
    if (B == 0) return BS_OK;
    if (!qkv || !kcache || !vcache || !cos || !sin || !pos || !out) return BS_ERR_NULL;
    if (!bs_aligned(qkv, 16) || !bs_aligned(kcache, 16) || !bs_aligned(vcache, 16) || !bs_aligned(cos, 16) ||
        !bs_aligned(sin, 16) || !bs_aligned(pos, 8) || !bs_aligned(out, 16))
        return BS_ERR_ALIGN;
    return bs_launch_attention_decode((const half_t *)qkv, (half_t *)kcache, (half_t *)vcache, (const half_t *)cos,
                                      (const half_t *)sin, pos, (half_t *)out, B, heads, kv_heads, head_dim, max_len,
                                      (hipStream_t)stream);
}

extern "C" int bs_argmax_f16(const void *x, int64_t *out, int B, int V, void *stream) {
    if (B < 0 || V <= 0) return BS_ERR_SHAPE;
    if (B == 0) return BS_OK;
    if (!x || !out) return BS_ERR_NULL;
    if (!bs_aligned(x, 16) || !bs_aligned(out, 8) || (B > 1 && V % 8 != 0)) return BS_ERR_ALIGN;
    return bs_launch_argmax((const half_t *)x, out, B, V, (hipStream_t)stream);
}

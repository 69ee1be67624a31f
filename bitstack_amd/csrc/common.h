// Shared host-side helpers for the gfx950 BitStack kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "../../include/bitstack_hip.h"

#define BS_VERSION_NUMBER 100  // 0.1.0

// Turn a failed HIP call into the documented negative status.
#define BS_HIP_TRY(expr)                                          \
    do {                                                          \
        hipError_t bs_e_ = (expr);                                \
        if (bs_e_ != hipSuccess) return BS_ERR_HIP_BASE - (int)bs_e_; \
    } while (0)

// A kernel launch reports configuration errors through hipGetLastError.
#define BS_LAUNCH_CHECK() BS_HIP_TRY(hipGetLastError())

static inline bool bs_aligned(const void *p, uintptr_t a) {
    return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0;
}

static inline int64_t bs_cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Kernels that need more than 64 KB of dynamic LDS must be allowed to, once per kernel AND
// per device (the attribute lives with the device's copy of the code).  `granted[d]` is the
// size already allowed on device d; the caller keeps one such array per kernel.
// Host threads may race here: the table entries are atomics (a torn read could skip a grant
// that was never made), and setting the attribute twice to the same or a larger size is harmless.
constexpr int BS_MAX_DEVICES = 64;
typedef std::atomic<size_t> bs_lds_grant;
static inline int bs_allow_lds(const void *kernel, size_t bytes, bs_lds_grant *granted) {
    if (bytes <= 64 * 1024) return BS_OK;
    int dev = 0;
    BS_HIP_TRY(hipGetDevice(&dev));
    const bool tracked = dev >= 0 && dev < BS_MAX_DEVICES;
    if (tracked && granted[dev].load(std::memory_order_acquire) >= bytes) return BS_OK;
    BS_HIP_TRY(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes));
    if (tracked) {
        size_t seen = granted[dev].load(std::memory_order_relaxed);
        while (seen < bytes && !granted[dev].compare_exchange_weak(seen, bytes, std::memory_order_release)) {}
    }
    return BS_OK;
}

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));
typedef uint32_t uint2_t __attribute__((ext_vector_type(2)));

// Internal launchers (one per translation unit), all return a status.
int bs_launch_reconstruct_packed(const uint8_t *packed, const half_t *u, const half_t *vt,
                                 half_t *w, int I, int M, int N, int K, hipStream_t s);
int bs_launch_linear_f16(const half_t *x, const half_t *w, const half_t *bias, half_t *y,
                         int T, int M, int N, hipStream_t s);
// the same product through hipBLASLt (dense_lt.hip); BS_ERR_SHAPE = not available for this call
constexpr int64_t BS_DENSE_LIBRARY_WORKSPACE = 64 << 20;
int bs_launch_linear_library(const half_t *x, const half_t *w, const half_t *bias, half_t *y, int T, int M, int N,
                             void *workspace, hipStream_t s);
int bs_launch_gemv(const uint8_t *packed, const half_t *u, const half_t *vt, const half_t *x,
                   const half_t *bias, half_t *y, int I, int M, int N, int K, int T,
                   void *workspace, int64_t workspace_bytes, hipStream_t s);
int64_t bs_gemv_workspace_bytes(int I, int M, int N, int K, int T);
void bs_gemv_plan_info(int I, int M, int N, int K, int T, int *waves, int *row_tiles_per_wave, int *grid, int *kmax);
int bs_gemv_plan_kernel(int I, int M, int N, int K, int T);
int bs_gemv_forward_path(int I, int M, int N, int K, int T);
int bs_gemv_set_kernel(int mode);
// epilogues of the grouped decode forward (values of BS_EPI_* in the public header)
enum { EPI_NONE = 0, EPI_RESIDUAL = 1, EPI_SWIGLU = 2 };
int64_t bs_gemv_group_workspace_bytes(const int *I, const int *M, int n, int N, int K, int T);
int bs_launch_gemv_group(int n, const uint8_t *const *packed, const half_t *const *u, const half_t *const *vt,
                         const half_t *const *bias, const int *I, const int *M, int N, int K, const half_t *x, int T,
                         int mode, const half_t *residual, half_t *y, int input_rms, float eps, void *workspace,
                         int64_t workspace_bytes, hipStream_t s);
// strip kernel (strip.hip): partial sums part[strip, t, m] of x . w^T with w rebuilt in registers
int bs_strip_partials(int I, int M, int N, int K, int T);
int bs_strip_kernel_choice(int I, int M, int N, int K, int T);
int bs_launch_strip_group(int n, const uint8_t *const *packed, const half_t *const *u, const half_t *const *vt,
                          const int *I, const int *M, float *const *part, float *ssq, const half_t *x,
                          int N, int K, int T, hipStream_t s);
// panel kernel (panel.hip): the same partial sums for up to 128 tokens, sign tiles decoded into LDS and
// multiplied on the matrix cores at once; bs_panel_partials = column groups (0: the shape is not taken)
constexpr int BS_PANEL_MAX_T = 128;
int bs_panel_partials(int I, int M, int N, int K, int T);
int bs_launch_panel(const uint8_t *packed, const half_t *u, const half_t *vt, int I, int M, float *part, const half_t *x,
                    int N, int K, int T, hipStream_t s);
// which kernel runs a forward of 49 tokens or more (bs_set_prefill_kernel, per thread): values of BS_PREFILL_*
int bs_prefill_mode();
// decode-step kernels around the linears (decode_step.hip)
int bs_launch_argmax(const half_t *x, int64_t *out, int B, int V, hipStream_t s);
int bs_launch_rmsnorm(const half_t *x, const half_t *weight, half_t *y, int T, int H, float eps, hipStream_t s);
int bs_launch_attention_decode(const half_t *qkv, half_t *kcache, half_t *vcache, const half_t *cos, const half_t *sin,
                               const int64_t *pos, half_t *out, int B, int heads, int kv_heads, int head_dim,
                               int max_len, hipStream_t s);

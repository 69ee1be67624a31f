// The dense product y[T, M] = x[T, N] @ w[M, N]^T (+ bias) through hipBLASLt: a COMPARATOR for tests
// and benchmarks, never chosen by bs_forward on its own (bs_set_dense_kernel(BS_DENSE_LIBRARY) asks for
// it per thread).  After the weight has been rebuilt the product is a plain fp16 GEMM with fp32
// accumulation, what the reference hands to F.linear (bitstack/modules/BitStackLinear.py:132,140,148)
// - which on ROCm is this library - so it is the yardstick linear_f16_kernel (gemm.hip) is timed against.
//
// hipBLASLt is opened at run time (dlopen of its SONAME), so libbitstack_hip.so has no link-time
// dependency on it.  In a process that already holds a copy (PyTorch ships one under the same SONAME)
// that copy is the one used.
//
// Row-major operands read as column-major ones: w is A = [N x M] (ld N, transposed), x is
// B = [N x T] (ld N), y is D = [M x T] (ld M); D = A^T B, bias broadcast along D's rows.
#include "common.h"

#include <dlfcn.h>
#include <hipblaslt/hipblaslt.h>

#include <map>
#include <mutex>
#include <tuple>

namespace {

struct LtApi {
    decltype(&hipblasLtCreate) create;
    decltype(&hipblasLtMatrixLayoutCreate) layout_create;
    decltype(&hipblasLtMatrixLayoutDestroy) layout_destroy;
    decltype(&hipblasLtMatmulDescCreate) desc_create;
    decltype(&hipblasLtMatmulDescDestroy) desc_destroy;
    decltype(&hipblasLtMatmulDescSetAttribute) desc_set;
    decltype(&hipblasLtMatmulPreferenceCreate) pref_create;
    decltype(&hipblasLtMatmulPreferenceSetAttribute) pref_set;
    decltype(&hipblasLtMatmulPreferenceDestroy) pref_destroy;
    decltype(&hipblasLtMatmulAlgoGetHeuristic) heuristic;
    decltype(&hipblasLtMatmul) matmul;
};

// One descriptor set and one chosen algorithm per (device, T, M, N, bias?).
struct LtPlan {
    hipblasLtMatmulDesc_t desc = nullptr;
    hipblasLtMatrixLayout_t a = nullptr, b = nullptr, d = nullptr;
    hipblasLtMatmulAlgo_t algo;
    size_t workspace = 0;
    bool usable = false;
};

// The plan table is bounded: a caller that sweeps prompt lengths would otherwise add an entry (and a
// heuristic query) per distinct token count for the life of the process.  When it is full it is emptied
// and rebuilt on demand - but only outside stream capture, where no graph can be recording the
// descriptors (a descriptor only lives on the host; recorded launches hold none of it).
constexpr size_t LT_MAX_PLANS = 256;

struct LtState {
    std::mutex mu;                    // one caller at a time: the bias pointer is an attribute of the shared descriptor
    bool tried = false;
    LtApi api{};
    bool loaded = false;
    hipblasLtHandle_t handle[BS_MAX_DEVICES] = {};
    std::map<std::tuple<int, int, int, int, int>, LtPlan> plans;
};
LtState g_lt;

template <class F>
bool resolve(void *so, const char *name, F &out) {
    out = reinterpret_cast<F>(dlsym(so, name));
    return out != nullptr;
}

bool load_api(LtState &st) {
    if (st.tried) return st.loaded;
    st.tried = true;
    void *so = dlopen("libhipblaslt.so.1", RTLD_NOW | RTLD_LOCAL);
    if (!so) return false;
    LtApi &a = st.api;
    st.loaded = resolve(so, "hipblasLtCreate", a.create) && resolve(so, "hipblasLtMatrixLayoutCreate", a.layout_create) &&
                resolve(so, "hipblasLtMatrixLayoutDestroy", a.layout_destroy) &&
                resolve(so, "hipblasLtMatmulDescCreate", a.desc_create) &&
                resolve(so, "hipblasLtMatmulDescDestroy", a.desc_destroy) &&
                resolve(so, "hipblasLtMatmulDescSetAttribute", a.desc_set) &&
                resolve(so, "hipblasLtMatmulPreferenceCreate", a.pref_create) &&
                resolve(so, "hipblasLtMatmulPreferenceSetAttribute", a.pref_set) &&
                resolve(so, "hipblasLtMatmulPreferenceDestroy", a.pref_destroy) &&
                resolve(so, "hipblasLtMatmulAlgoGetHeuristic", a.heuristic) && resolve(so, "hipblasLtMatmul", a.matmul);
    return st.loaded;
}

void destroy_plan(const LtApi &a, LtPlan &p) {
    if (p.a) a.layout_destroy(p.a);
    if (p.b) a.layout_destroy(p.b);
    if (p.d) a.layout_destroy(p.d);
    if (p.desc) a.desc_destroy(p.desc);
    p = LtPlan{};
}

bool fill_plan(LtState &st, hipblasLtHandle_t h, LtPlan &p, int T, int M, int N, bool bias) {
    const LtApi &a = st.api;
    const auto ok = [](hipblasStatus_t s) { return s == HIPBLAS_STATUS_SUCCESS; };
    if (!ok(a.desc_create(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F))) return false;
    const int32_t op_t = HIPBLAS_OP_T, op_n = HIPBLAS_OP_N;
    if (!ok(a.desc_set(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &op_t, sizeof(op_t))) ||
        !ok(a.desc_set(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &op_n, sizeof(op_n))))
        return false;
    if (bias) {
        const uint32_t epi = HIPBLASLT_EPILOGUE_BIAS;
        const int32_t bias_type = HIP_R_16F;
        const void *none = nullptr;       // the real pointer is set per call; the heuristic only needs the epilogue
        if (!ok(a.desc_set(p.desc, HIPBLASLT_MATMUL_DESC_EPILOGUE, &epi, sizeof(epi))) ||
            !ok(a.desc_set(p.desc, HIPBLASLT_MATMUL_DESC_BIAS_DATA_TYPE, &bias_type, sizeof(bias_type))) ||
            !ok(a.desc_set(p.desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &none, sizeof(none))))
            return false;
    }
    if (!ok(a.layout_create(&p.a, HIP_R_16F, (uint64_t)N, (uint64_t)M, N)) ||
        !ok(a.layout_create(&p.b, HIP_R_16F, (uint64_t)N, (uint64_t)T, N)) ||
        !ok(a.layout_create(&p.d, HIP_R_16F, (uint64_t)M, (uint64_t)T, M)))
        return false;
    hipblasLtMatmulPreference_t pref = nullptr;
    if (!ok(a.pref_create(&pref))) return false;
    const uint64_t max_ws = BS_DENSE_LIBRARY_WORKSPACE;
    bool found = ok(a.pref_set(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &max_ws, sizeof(max_ws)));
    if (found) {
        hipblasLtMatmulHeuristicResult_t res{};
        int n = 0;
        found = ok(a.heuristic(h, p.desc, p.a, p.b, p.d, p.d, pref, 1, &res, &n)) && n >= 1 &&
                res.state == HIPBLAS_STATUS_SUCCESS && res.workspaceSize <= max_ws;
        if (found) {
            p.algo = res.algo;
            p.workspace = res.workspaceSize;
        }
    }
    a.pref_destroy(pref);
    return found;
}

// A plan that cannot be completed leaves nothing behind but the (empty) table entry that says so.
void make_plan(LtState &st, hipblasLtHandle_t h, LtPlan &p, int T, int M, int N, bool bias) {
    if (fill_plan(st, h, p, T, M, N, bias)) {
        p.usable = true;
    } else {
        destroy_plan(st.api, p);
    }
}

}  // namespace

// BS_OK: the product has been enqueued.  BS_ERR_SHAPE: declined BEFORE anything was enqueued - hipBLASLt is
// not installed, has no kernel for the shape, the buffers are not aligned for it, or the shape is new
// while its stream is being captured (setting the library up is host work that may allocate) - and the
// caller runs its own kernel.  Anything else is a failure after the call had been accepted (a HIP
// status, or BS_ERR_LIBRARY for a hipBLASLt one): final, the caller must not paper over it.
// `workspace` holds BS_DENSE_LIBRARY_WORKSPACE bytes, 256-byte aligned.
int bs_launch_linear_library(const half_t *x, const half_t *w, const half_t *bias, half_t *y, int T, int M, int N,
                             void *workspace, hipStream_t s) {
    if (!bs_aligned(x, 16) || !bs_aligned(w, 16) || !bs_aligned(y, 16) || N % 8 != 0 || M % 8 != 0) return BS_ERR_SHAPE;
    int dev = -1;
    BS_HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= BS_MAX_DEVICES) return BS_ERR_SHAPE;
    LtState &st = g_lt;
    std::lock_guard<std::mutex> lock(st.mu);
    const auto key = std::make_tuple(dev, T, M, N, bias ? 1 : 0);
    auto it = st.plans.find(key);
    if (it == st.plans.end()) {
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        BS_HIP_TRY(hipStreamIsCapturing(s, &cap));
        if (cap != hipStreamCaptureStatusNone) return BS_ERR_SHAPE;
        if (!load_api(st)) return BS_ERR_SHAPE;
        if (!st.handle[dev] && st.api.create(&st.handle[dev]) != HIPBLAS_STATUS_SUCCESS) {
            st.handle[dev] = nullptr;
            return BS_ERR_SHAPE;
        }
        if (st.plans.size() >= LT_MAX_PLANS) {
            for (auto &kv : st.plans) destroy_plan(st.api, kv.second);
            st.plans.clear();
        }
        LtPlan p;
        make_plan(st, st.handle[dev], p, T, M, N, bias != nullptr);
        it = st.plans.emplace(key, p).first;
    }
    LtPlan &p = it->second;
    if (!p.usable) return BS_ERR_SHAPE;
    if (bias) {
        const void *bp = bias;
        if (st.api.desc_set(p.desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bp, sizeof(bp)) != HIPBLAS_STATUS_SUCCESS)
            return BS_ERR_LIBRARY;
    }
    const float alpha = 1.f, beta = 0.f;
    const hipblasStatus_t r = st.api.matmul(st.handle[dev], p.desc, &alpha, w, p.a, x, p.b, &beta, y, p.d, y, p.d, &p.algo,
                                            workspace, p.workspace, s);
    return r == HIPBLAS_STATUS_SUCCESS ? BS_OK : BS_ERR_LIBRARY;
}

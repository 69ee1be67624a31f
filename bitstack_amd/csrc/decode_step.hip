// The two steps of a decoder layer that sit between the compressed linears at
// decode time: RMSNorm, and one position of rotary grouped-query attention over a
// static KV cache.  Small, latency-bound kernels; their point is to replace a
// dozen framework launches per layer by two.
#include "common.h"

namespace {

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

// One workgroup per row; the row stays in registers between the two passes.
constexpr int RMS_THREADS = 256, RMS_MAX_CHUNKS = 8;   // 256 * 8 * 8 halves = 16384 columns

__global__ __launch_bounds__(RMS_THREADS) void rmsnorm_kernel(const half_t *__restrict__ x,
                                                              const half_t *__restrict__ weight,
                                                              half_t *__restrict__ y, int H, float eps) {
    __shared__ float wsum[RMS_THREADS / 64];
    const int tid = threadIdx.x;
    const half_t *xr = x + (int64_t)blockIdx.x * H;
    half_t *yr = y + (int64_t)blockIdx.x * H;
    half8_t v[RMS_MAX_CHUNKS];
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < RMS_MAX_CHUNKS; c++) {
        const int col = (c * RMS_THREADS + tid) * 8;
        if (col < H) {
            v[c] = *reinterpret_cast<const half8_t *>(xr + col);
#pragma unroll
            for (int e = 0; e < 8; e++) ss += (float)v[c][e] * (float)v[c][e];
        }
    }
    ss = wave_sum(ss);
    if ((tid & 63) == 0) wsum[tid >> 6] = ss;
    __syncthreads();
    float total = 0.f;
#pragma unroll
    for (int w = 0; w < RMS_THREADS / 64; w++) total += wsum[w];
    const float r = rsqrtf(total / (float)H + eps);
#pragma unroll
    for (int c = 0; c < RMS_MAX_CHUNKS; c++) {
        const int col = (c * RMS_THREADS + tid) * 8;
        if (col < H) {
            const half8_t w8 = *reinterpret_cast<const half8_t *>(weight + col);
            half8_t o;
#pragma unroll
            for (int e = 0; e < 8; e++) o[e] = (half_t)((float)(half_t)((float)v[c][e] * r) * (float)w8[e]);
            *reinterpret_cast<half8_t *>(yr + col) = o;
        }
    }
}

// One workgroup per (query head, sequence).  1024 threads = 64 groups of 16 lanes;
// a group walks every 64th cached position, a lane owns 8 of the 128 dimensions
// (one 16-byte load per cached row and lane, a row is one contiguous 256 bytes).
// One pass: k and v of four positions are fetched together and folded into a
// running (max, sum, weighted v) per group; the 64 groups are merged through LDS.
constexpr int ATT_THREADS = 1024, ATT_GROUPS = ATT_THREADS / 16, ATT_D = 128, ATT_MAX_LEN = 8192;

__global__ __launch_bounds__(ATT_THREADS) void attention_decode_kernel(
    const half_t *__restrict__ qkv, half_t *__restrict__ kcache, half_t *__restrict__ vcache,
    const half_t *__restrict__ cosv, const half_t *__restrict__ sinv, const int64_t *__restrict__ pos_ptr,
    half_t *__restrict__ out, int heads, int kv_heads, int max_len) {
    __shared__ float qs[ATT_D];                  // rotated query, pre-scaled
    __shared__ __attribute__((aligned(16))) half_t knew[ATT_D], vnew[ATT_D];   // this position's rotated k and v
    __shared__ float gm[ATT_GROUPS], gl[ATT_GROUPS];             // per group: running max, sum of exp
    __shared__ float accs[ATT_GROUPS][ATT_D];
    const int tid = threadIdx.x, lane16 = tid & 15, grp = tid >> 4;
    const int head = blockIdx.x, b = blockIdx.y;
    const int rep = heads / kv_heads, hk = head / rep;
    const int row = (heads + 2 * kv_heads) * ATT_D;
    const half_t *q = qkv + (int64_t)b * row + head * ATT_D;
    const half_t *kn = qkv + (int64_t)b * row + (heads + hk) * ATT_D;
    const half_t *vn = qkv + (int64_t)b * row + (heads + kv_heads + hk) * ATT_D;
    half_t *orow = out + ((int64_t)b * heads + head) * ATT_D;
    // what does not depend on the position is fetched before the position is known
    float qa = 0.f, qb = 0.f, ka = 0.f, kb = 0.f;
    half_t vv = (half_t)0;
    if (tid < ATT_D / 2) {
        qa = (float)q[tid]; qb = (float)q[tid + ATT_D / 2];
        ka = (float)kn[tid]; kb = (float)kn[tid + ATT_D / 2];
    } else if (tid < ATT_D / 2 + ATT_D) {
        vv = vn[tid - ATT_D / 2];
    }
    const int64_t pos64 = *pos_ptr;
    if (pos64 < 0 || pos64 >= max_len) {         // nothing sensible to do: defined output, no access outside the cache
        if (tid < ATT_D) orow[tid] = (half_t)0;
        return;
    }
    const int pos = (int)pos64;
    half_t *kc = kcache + ((int64_t)b * kv_heads + hk) * max_len * ATT_D;
    half_t *vc = vcache + ((int64_t)b * kv_heads + hk) * max_len * ATT_D;

    if (tid < ATT_D / 2) {
        const float c = (float)cosv[(int64_t)pos * (ATT_D / 2) + tid], s = (float)sinv[(int64_t)pos * (ATT_D / 2) + tid];
        const float scale = 0.08838834764831845f;       // 1 / sqrt(128)
        qs[tid] = (float)(half_t)(qa * c - qb * s) * scale;
        qs[tid + ATT_D / 2] = (float)(half_t)(qb * c + qa * s) * scale;
        knew[tid] = (half_t)(ka * c - kb * s);
        knew[tid + ATT_D / 2] = (half_t)(kb * c + ka * s);
    } else if (tid < ATT_D / 2 + ATT_D) {
        vnew[tid - ATT_D / 2] = vv;
    }
    __syncthreads();
    if (head % rep == 0 && tid < ATT_D) {        // one head of the group appends to the cache
        kc[(int64_t)pos * ATT_D + tid] = knew[tid];
        vc[(int64_t)pos * ATT_D + tid] = vnew[tid];
    }

    float qreg[8];
#pragma unroll
    for (int e = 0; e < 8; e++) qreg[e] = qs[8 * lane16 + e];
    float m = -INFINITY, l = 0.f;
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    auto score_of = [&](const half8_t k8) {
        float d = 0.f;
#pragma unroll
        for (int e = 0; e < 8; e++) d += qreg[e] * (float)k8[e];
#pragma unroll
        for (int o = 8; o >= 1; o >>= 1) d += __shfl_xor(d, o, 64);
        return d;                                 // the same value in all 16 lanes of the group
    };
    auto fold = [&](float sc, const half8_t v8) {
        const float mn = fmaxf(m, sc);
        const float r = __expf(m - mn), w = __expf(sc - mn);      // exp(-inf) = 0 on the first position
        l = l * r + w;
#pragma unroll
        for (int e = 0; e < 8; e++) acc[e] = acc[e] * r + w * (float)v8[e];
        m = mn;
    };
    for (int p0 = grp; p0 < pos; p0 += 4 * ATT_GROUPS) {
        half8_t k8[4], v8[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int p = min(p0 + ATT_GROUPS * j, pos - 1);
            k8[j] = *reinterpret_cast<const half8_t *>(kc + (int64_t)p * ATT_D + 8 * lane16);
            v8[j] = *reinterpret_cast<const half8_t *>(vc + (int64_t)p * ATT_D + 8 * lane16);
        }
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const float sc = score_of(k8[j]);
            if (p0 + ATT_GROUPS * j < pos) fold(sc, v8[j]);
        }
    }
    if (grp == 0)      // this step's own k and v, from LDS
        fold(score_of(*reinterpret_cast<const half8_t *>(knew + 8 * lane16)),
             *reinterpret_cast<const half8_t *>(vnew + 8 * lane16));
    if (lane16 == 0) { gm[grp] = m; gl[grp] = l; }
#pragma unroll
    for (int e = 0; e < 8; e++) accs[grp][8 * lane16 + e] = acc[e];
    __syncthreads();
    if (tid < ATT_D) {
        float mx = gm[0];
#pragma unroll
        for (int gq = 1; gq < ATT_GROUPS; gq++) mx = fmaxf(mx, gm[gq]);
        float o = 0.f, den = 0.f;
#pragma unroll
        for (int gq = 0; gq < ATT_GROUPS; gq++) {
            const float r = gl[gq] > 0.f ? __expf(gm[gq] - mx) : 0.f;     // groups that saw no position
            o += r * accs[gq][tid];
            den += r * gl[gq];
        }
        orow[tid] = (half_t)(o / den);
    }
}

// Grouped-query variant for long caches: one workgroup serves REP query heads that share a
// KV head, so a cached row is fetched once for REP heads (the fetches, not the arithmetic,
// are what a long cache costs).  1024 threads = 64 groups of 16 lanes; a group walks every
// 64th position, a lane owns 8 of the 128 dimensions.  The rotated queries stay in registers as fp16 pairs and the scores
// are v_dot2_f32_f16 sums (fp16 products, fp32 accumulation) reduced over the 16 lanes with
// DPP adds; the softmax runs in base 2 (log2(e) folded into the score scale).  Per head a
// running (max, sum, weighted v); groups are merged by shuffles inside a wave, waves through LDS.
constexpr int GQA_THREADS = 1024, GQA_WAVES = GQA_THREADS / 64;

// sum over the 16 lanes of a DPP row (every lane ends with the total)
__device__ __forceinline__ float row_sum16(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));   // quad_perm [2,3,0,1]
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));  // row_half_mirror
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true));  // row_mirror
    return v;
}

template <int REP>
__global__ __launch_bounds__(GQA_THREADS) void attention_decode_gqa_kernel(
    const half_t *__restrict__ qkv, half_t *__restrict__ kcache, half_t *__restrict__ vcache,
    const half_t *__restrict__ cosv, const half_t *__restrict__ sinv, const int64_t *__restrict__ pos_ptr,
    half_t *__restrict__ out, int heads, int kv_heads, int max_len) {
    __shared__ __attribute__((aligned(16))) half_t qrot[REP][ATT_D];           // rotated queries
    __shared__ __attribute__((aligned(16))) half_t knew[ATT_D], vnew[ATT_D];   // this position's rotated k and v
    __shared__ float wm[REP][GQA_WAVES], wl[REP][GQA_WAVES];
    __shared__ float wacc[REP][GQA_WAVES][ATT_D];
    const int tid = threadIdx.x, lane16 = tid & 15, grp = tid >> 4, wave = tid >> 6;
    const int head0 = blockIdx.x * REP, b = blockIdx.y;          // this workgroup's first query head
    const int rep = heads / kv_heads, hk = head0 / rep;          // REP divides rep: all REP heads share KV head hk
    const int row = (heads + 2 * kv_heads) * ATT_D;
    const half_t *qb_ = qkv + (int64_t)b * row + (int64_t)head0 * ATT_D;        // the REP query heads, contiguous
    const half_t *kn = qkv + (int64_t)b * row + (heads + hk) * ATT_D;
    const half_t *vn = qkv + (int64_t)b * row + (heads + kv_heads + hk) * ATT_D;
    // Work items of the set-up: REP * 64 query pairs, 64 key pairs (dimension i and i + 64 rotate
    // together), 128 values; at most two per thread.  What does not depend on the position is
    // fetched before the position is known.
    constexpr int QP = REP * 64, ITEMS = QP + 64 + ATT_D;
    static_assert(ITEMS <= 2 * GQA_THREADS, "two set-up items per thread");
    float fa[2] = {0.f, 0.f}, fb[2] = {0.f, 0.f};
#pragma unroll
    for (int k = 0; k < 2; k++) {
        const int it = tid + k * GQA_THREADS;
        if (it < QP) {
            const int h = it >> 6, i = it & 63;
            fa[k] = (float)qb_[h * ATT_D + i]; fb[k] = (float)qb_[h * ATT_D + i + 64];
        } else if (it < QP + 64) {
            fa[k] = (float)kn[it - QP]; fb[k] = (float)kn[it - QP + 64];
        } else if (it < ITEMS) {
            fa[k] = (float)vn[it - QP - 64];
        }
    }
    const int64_t pos64 = *pos_ptr;
    if (pos64 < 0 || pos64 >= max_len) {         // nothing sensible to do: defined output, no access outside the cache
        for (int it = tid; it < REP * ATT_D; it += GQA_THREADS)
            out[((int64_t)b * heads + head0) * ATT_D + it] = (half_t)0;
        return;
    }
    const int pos = (int)pos64;
    half_t *kc = kcache + ((int64_t)b * kv_heads + hk) * max_len * ATT_D;
    half_t *vc = vcache + ((int64_t)b * kv_heads + hk) * max_len * ATT_D;
#pragma unroll
    for (int k = 0; k < 2; k++) {
        const int it = tid + k * GQA_THREADS;
        if (it < QP + 64) {
            const int i = it & 63;
            const float c = (float)cosv[(int64_t)pos * (ATT_D / 2) + i], sn = (float)sinv[(int64_t)pos * (ATT_D / 2) + i];
            const half_t lo = (half_t)(fa[k] * c - fb[k] * sn), hi = (half_t)(fb[k] * c + fa[k] * sn);
            if (it < QP) { qrot[it >> 6][i] = lo; qrot[it >> 6][i + 64] = hi; }
            else { knew[i] = lo; knew[i + 64] = hi; }
        } else if (it < ITEMS) {
            vnew[it - QP - 64] = (half_t)fa[k];
        }
    }
    __syncthreads();
    if (head0 % rep == 0 && tid < ATT_D) {       // one workgroup of the KV head appends this position to the cache
        kc[(int64_t)pos * ATT_D + tid] = knew[tid];
        vc[(int64_t)pos * ATT_D + tid] = vnew[tid];
    }

    half2_t qreg[REP][4];                        // this lane's 8 dimensions of every query
#pragma unroll
    for (int h = 0; h < REP; h++)
#pragma unroll
        for (int e = 0; e < 4; e++) qreg[h][e] = *reinterpret_cast<const half2_t *>(&qrot[h][8 * lane16 + 2 * e]);
    const float scale2 = 0.08838834764831845f * 1.4426950408889634f;    // 1 / sqrt(128) * log2(e)
    float m[REP], l[REP], acc[REP][8];
#pragma unroll
    for (int h = 0; h < REP; h++) {
        m[h] = -INFINITY;
        l[h] = 0.f;
#pragma unroll
        for (int e = 0; e < 8; e++) acc[h][e] = 0.f;
    }
    auto fold = [&](const half8_t k8, const half8_t v8) {
        float vf[8];
#pragma unroll
        for (int e = 0; e < 8; e++) vf[e] = (float)v8[e];
#pragma unroll
        for (int h = 0; h < REP; h++) {
            float d = 0.f;
#pragma unroll
            for (int e = 0; e < 4; e++)
                d = __builtin_amdgcn_fdot2(qreg[h][e], (half2_t){k8[2 * e], k8[2 * e + 1]}, d, false);
            const float sc = row_sum16(d) * scale2;                  // the same value in all 16 lanes of the group
            const float mn = fmaxf(m[h], sc);
            const float r = __builtin_amdgcn_exp2f(m[h] - mn), w = __builtin_amdgcn_exp2f(sc - mn);   // exp2(-inf) = 0 on the first position
            l[h] = l[h] * r + w;
#pragma unroll
            for (int e = 0; e < 8; e++) acc[h][e] = acc[h][e] * r + w * vf[e];
            m[h] = mn;
        }
    };
    constexpr int GROUPS = GQA_THREADS / 16;
    for (int p0 = grp; p0 < pos; p0 += 4 * GROUPS) {
        half8_t k8[4], v8[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int p = min(p0 + GROUPS * j, pos - 1);
            k8[j] = *reinterpret_cast<const half8_t *>(kc + (int64_t)p * ATT_D + 8 * lane16);
            v8[j] = *reinterpret_cast<const half8_t *>(vc + (int64_t)p * ATT_D + 8 * lane16);
        }
#pragma unroll
        for (int j = 0; j < 4; j++)
            if (p0 + GROUPS * j < pos) fold(k8[j], v8[j]);
    }
    if (grp == 0)      // this step's own k and v, from LDS
        fold(*reinterpret_cast<const half8_t *>(knew + 8 * lane16), *reinterpret_cast<const half8_t *>(vnew + 8 * lane16));

    // the four groups of a wave (lanes 16 and 32 apart), then the waves through LDS
#pragma unroll
    for (int h = 0; h < REP; h++) {
#pragma unroll
        for (int o = 16; o <= 32; o <<= 1) {
            const float m2 = __shfl_xor(m[h], o, 64), l2 = __shfl_xor(l[h], o, 64);
            const float mn = fmaxf(m[h], m2);
            const float r1 = mn == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m[h] - mn);
            const float r2 = mn == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m2 - mn);
            l[h] = l[h] * r1 + l2 * r2;
#pragma unroll
            for (int e = 0; e < 8; e++) acc[h][e] = acc[h][e] * r1 + __shfl_xor(acc[h][e], o, 64) * r2;
            m[h] = mn;
        }
        if ((tid & 63) == 0) { wm[h][wave] = m[h]; wl[h][wave] = l[h]; }
        if ((tid & 63) < 16) {
#pragma unroll
            for (int e = 0; e < 8; e++) wacc[h][wave][8 * lane16 + e] = acc[h][e];
        }
    }
    __syncthreads();
    for (int it = tid; it < REP * ATT_D; it += GQA_THREADS) {
        const int h = it >> 7, dim = it & (ATT_D - 1);
        float mx = wm[h][0];
#pragma unroll
        for (int w = 1; w < GQA_WAVES; w++) mx = fmaxf(mx, wm[h][w]);
        float o = 0.f, den = 0.f;
#pragma unroll
        for (int w = 0; w < GQA_WAVES; w++) {
            const float r = wl[h][w] > 0.f ? __builtin_amdgcn_exp2f(wm[h][w] - mx) : 0.f;     // waves that saw no position
            o += r * wacc[h][w][dim];
            den += r * wl[h][w];
        }
        out[((int64_t)b * heads + head0 + h) * ATT_D + dim] = (half_t)(o / den);
    }
}

// Greedy token: index of the largest of V fp16 values per row (the lowest index among
// equals; NaN never wins), one workgroup per row.
constexpr int ARG_THREADS = 1024;

__global__ __launch_bounds__(ARG_THREADS) void argmax_kernel(const half_t *__restrict__ x, int64_t *__restrict__ out, int V) {
    __shared__ float bv[ARG_THREADS / 64];
    __shared__ int bi[ARG_THREADS / 64];
    const int tid = threadIdx.x;
    const half_t *row = x + (int64_t)blockIdx.x * V;
    float best = -INFINITY;
    int at = 0x7fffffff;
    const int v8 = V & ~7;
    for (int c = tid * 8; c < v8; c += ARG_THREADS * 8) {       // ascending per thread: a later equal value never replaces
        const half8_t v = *reinterpret_cast<const half8_t *>(row + c);
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const float f = (float)v[e];
            if (f > best || (f == best && c + e < at)) { best = f; at = c + e; }
        }
    }
    for (int c = v8 + tid; c < V; c += ARG_THREADS) {
        const float f = (float)row[c];
        if (f > best || (f == best && c < at)) { best = f; at = c; }
    }
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) {
        const float ob = __shfl_xor(best, o, 64);
        const int oa = __shfl_xor(at, o, 64);
        if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
    }
    if ((tid & 63) == 0) { bv[tid >> 6] = best; bi[tid >> 6] = at; }
    __syncthreads();
    if (tid == 0) {
        for (int w = 1; w < ARG_THREADS / 64; w++)
            if (bv[w] > best || (bv[w] == best && bi[w] < at)) { best = bv[w]; at = bi[w]; }
        out[blockIdx.x] = at == 0x7fffffff ? 0 : at;            // a row of NaNs / -inf: index 0
    }
}

}  // namespace

int bs_launch_argmax(const half_t *x, int64_t *out, int B, int V, hipStream_t s) {
    argmax_kernel<<<B, ARG_THREADS, 0, s>>>(x, out, V);
    BS_LAUNCH_CHECK();
    return BS_OK;
}

int bs_launch_rmsnorm(const half_t *x, const half_t *weight, half_t *y, int T, int H, float eps, hipStream_t s) {
    if (H > RMS_THREADS * RMS_MAX_CHUNKS * 8) return BS_ERR_SHAPE;
    rmsnorm_kernel<<<T, RMS_THREADS, 0, s>>>(x, weight, y, H, eps);
    BS_LAUNCH_CHECK();
    return BS_OK;
}

int bs_launch_attention_decode(const half_t *qkv, half_t *kcache, half_t *vcache, const half_t *cos, const half_t *sin,
                               const int64_t *pos, half_t *out, int B, int heads, int kv_heads, int head_dim,
                               int max_len, hipStream_t s) {
    if (head_dim != ATT_D || max_len > ATT_MAX_LEN) return BS_ERR_SHAPE;
    // Long caches and more (head, sequence) pairs than CUs: four (or two) query heads of a KV
    // head per workgroup, a quarter (half) of the cache fetches.  A workgroup of the grouped
    // kernel takes longer than one of the per-head kernel (3000 positions: 55 us against 25),
    // so it only pays once the per-head kernel would need more than one round of workgroups
    // (8 sequences x 64 heads at 2100 positions: 45 us against 79).
    const int rep = heads / kv_heads;
    const bool grouped = max_len >= 1024 && (int64_t)B * heads > 256;
    if (grouped && rep % 4 == 0)
        attention_decode_gqa_kernel<4><<<dim3(heads / 4, B), GQA_THREADS, 0, s>>>(qkv, kcache, vcache, cos, sin, pos, out,
                                                                                 heads, kv_heads, max_len);
    else if (grouped && rep % 2 == 0)
        attention_decode_gqa_kernel<2><<<dim3(heads / 2, B), GQA_THREADS, 0, s>>>(qkv, kcache, vcache, cos, sin, pos, out,
                                                                                 heads, kv_heads, max_len);
    else
        attention_decode_kernel<<<dim3(heads, B), ATT_THREADS, 0, s>>>(qkv, kcache, vcache, cos, sin, pos, out, heads,
                                                                      kv_heads, max_len);
    BS_LAUNCH_CHECK();
    return BS_OK;
}

// Weight reconstruction for gfx950:
//   w[m, n] = fp16( sum_i s_i[m, n] * sum_r u_i[m, r] * vt_i[r, n] )
// fp32 everywhere until the single final rounding.
//
// Tiled kernel.  A workgroup owns a strip of 128 columns and a range of rows.
// It first stages the strip's slice of vt for ALL blocks in LDS, transposed to
// [block][column][rank] (vt is stored rank-major, the MFMA wants the rank
// index contiguous per lane; 16 halves per column plus 4 after every 8 columns keeps
// the 8-byte fragment reads aligned and off each other's banks), then walks its rows 16 per wave at a time with
// no further barrier.  Per block the rank-k product of a 16 x 16 patch is one
// v_mfma_f32_16x16x16_f16 computed TRANSPOSED, D[n, m] = sum_r vt[r, n] u[m, r],
// so that a lane ends up with four consecutive columns of one row - one nibble
// of that row's packed sign byte - and, over a pair of patches, with a whole byte
// (eight consecutive columns, one 16-byte store).  A nibble addresses a 16-entry
// table in LDS that holds its four signs as halves of +-1.0, which a mixed-precision
// FMA (fp32 product x fp16 sign + fp32 sum) multiplies in: half a VALU instruction per
// sign for the lookup instead of two for shifting and merging each sign bit.  Signs and u of the
// next block are loaded while the current block is multiplied.
#include "common.h"

#include <type_traits>

namespace {

constexpr int RT_COLS = 128;   // columns per workgroup strip
constexpr int VSTRIDE = 16;    // halves per column in LDS: the 16 ranks, contiguous
constexpr int VGROUP_PAD = 4;  // extra halves after every 8 columns (keeps the fragment reads off each other's banks)
constexpr int VBLOCK = RT_COLS * VSTRIDE + (RT_COLS / 8) * VGROUP_PAD;   // halves per block in LDS
constexpr int RT_MAXB = 36;    // most blocks whose vt strip fits in LDS (36 x 4.1 KB)
constexpr int SIGN_LUT_HALVES = 64;   // 16 nibbles x 4 signs

// K16: the rank is 16 (every u fragment is one 8-byte load).  Smaller ranks pick their halves one by one behind
// branches, and the compiler then waits for every load in flight where the branches meet: that instantiation runs
// one pair ahead at best.
template <bool PACKED, bool K16>
__global__ __launch_bounds__(256, 4) void reconstruct_tile_kernel(
    const uint8_t *__restrict__ packed, const int8_t *__restrict__ sign,
    const half_t *__restrict__ u, const half_t *__restrict__ vt, half_t *__restrict__ w,
    int I, int M, int N, int K, int rows_per_wg) {
    // First the 16 sign nibbles as four halves each (+1.0 for a set bit, first column in the top bit; at offset 0, so
    // that a nibble times 8 is the address), then [I][VBLOCK]: column c of a block at c * 16 + (c / 8) * 4.
    extern __shared__ __attribute__((aligned(128))) half_t lds_all[];
    half_t *const lut = lds_all;
    half_t *const vl = lds_all + SIGN_LUT_HALVES;
    // the table's LDS address as a number: the table is 128-byte aligned, so a nibble's offset is OR-ed into it
    typedef const __attribute__((address_space(3))) half4_t *lds_half4_ptr;
    const uint32_t lut_base = (uint32_t)reinterpret_cast<uintptr_t>((const __attribute__((address_space(3))) half_t *)lut);

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // the same in every lane: loop counts that depend on it stay scalar
    const int lm = lane & 15, g = lane >> 4;
    // Workgroups are dealt round-robin to the 8 XCDs, each with its own L2.  The eight
    // strips that share one 128-byte line of sign bytes must meet in ONE L2, and so
    // should the row groups that re-read one strip of vt: every XCD gets a contiguous
    // run of slots ordered (octet of strips, row group, strip within the octet).  The
    // grid is padded to whole octets; slots beyond the last strip do nothing.
    int n0, row_begin;
    {
        const int nb = gridDim.x * gridDim.y, lin = blockIdx.x + gridDim.x * blockIdx.y;
        const int xcd = lin & 7, loc = lin >> 3, base = nb >> 3, rem = nb & 7;
        const int v = xcd * base + min(xcd, rem) + loc;
        const int rest = v >> 3, strip = (rest / (int)gridDim.y) * 8 + (v & 7);
        if (strip * RT_COLS >= N) return;
        n0 = strip * RT_COLS;
        row_begin = (rest % (int)gridDim.y) * rows_per_wg;
    }
    const int row_end = min(row_begin + rows_per_wg, M);
    const int64_t row_bytes = N >> 3;
    const int64_t block_bytes = (int64_t)M * row_bytes;

    // staging role: rank index fastest across lanes, 16 pieces of 8 columns
    const int sr = tid & 15, sp = tid >> 4;
    // Patches come in pairs: of a 32-column group, patch 2q takes columns 8g'..8g'+3 and patch
    // 2q+1 columns 8g'+4..8g'+7 (g' = 0..3), so that a lane (row lm, group g) ends up with EIGHT
    // consecutive columns of its row - one byte of the packed signs, one 16-byte store.
    // The lane's byte of a sign word is byte g; its two nibbles, times 8, address the table:
    // (word >> sh_hi) & 0x78 for the first four columns, (word rotated right by sh_lo) & 0x78 for the others.
    const int sh_hi = 8 * g + 1, sh_lo = (8 * g - 3) & 31;
    // this lane's A-fragment column within a 32-column group (n-index lm of either patch, less 4 * (s & 1))
    const int acol = 8 * (lm >> 2) + (lm & 3);
    const int aoff = acol * VSTRIDE + (lm >> 2) * VGROUP_PAD + 4 * g;

    {
        const int i0 = 0, ib = I;
        // u rows and sign words of one (row step, block); requested one block ahead, also
        // across the end of a row step (first block of the next 16 rows), and issued for
        // the very first block before the vt strip is staged
        // Addresses are a wave-uniform 64-bit base (the block: scalar arithmetic) plus a 32-bit
        // offset per lane that depends on the row only and is renewed once per row step.
        uint32_t off_u;                             // bytes: this lane's u row (its four ranks)
        auto load_u = [&](int i, half4_t &b) {
            const char *ub = reinterpret_cast<const char *>(u) + (int64_t)i * M * K * 2;
            const half_t *up = reinterpret_cast<const half_t *>(ub + off_u);
            if (K16) {
                b = *reinterpret_cast<const half4_t *>(up);
            } else {
#pragma unroll
                for (int j = 0; j < 4; j++) b[j] = (4 * g + j < K) ? up[j] : (half_t)0;
            }
        };
        // The (row step, block) pairs of this wave form one sequence.  u rows are requested pair by pair, three pairs
        // ahead, into four register sets used in turn (the loop is written out eight pairs at a time, so that no set is
        // ever copied into another: a copy waits for the load it copies).  Sign words are requested FOUR PAIRS PER
        // INSTRUCTION: lane group g loads the 16 bytes of pair 4 q + g of the sequence (its row's sign bytes of this
        // strip in that pair's block), and the pair that is being multiplied fetches its words from the group that
        // holds them with four cross-lane reads.  Loaded pair by pair, all four lane groups requested the same 16
        // bytes per row, and a load instruction costs the memory pipeline its 16 rows' lines whatever it brings.
        half4_t b_set[4];
        uint4_t quad[2];
        const int first_row = row_begin + wave * 16;
        // Requests are unconditional (behind the last pair they repeat its row step): a
        // branch around a load makes the compiler wait for every load in flight at the join.
        const int last_m0 = first_row + ((max(row_end - first_row, 1) - 1) / 64) * 64;
        int pf_i = 0, pf_m0 = first_row;           // the pair the next u request is for
        auto set_row = [&](int m0) {
            const int row = min(min(m0, last_m0) + lm, M - 1);
            off_u = (uint32_t)(row * K + 4 * g) * 2u;
        };
        set_row(pf_m0);
        auto request_u = [&](half4_t &b) {
            load_u(i0 + pf_i, b);
            if (++pf_i == ib) {
                pf_i = 0;
                pf_m0 += 64;
                set_row(pf_m0);
            }
        };
        // the pair this lane loads for the next quad: block ql_i of the row step at ql_m0 (per lane: the groups differ)
        int ql_i = g, ql_m0 = first_row;
        auto wrap_quad = [&]() {
#pragma unroll
            for (int r = 0; r < 4; r++)
                if (ql_i >= ib) {
                    ql_i -= ib;
                    ql_m0 += 64;
                }
        };
        wrap_quad();
        auto request_quad = [&](uint4_t &qd) {
            if (PACKED) {
                const int row = min(min(ql_m0, last_m0) + lm, M - 1);
                qd = *reinterpret_cast<const uint4_t *>(packed + (int64_t)(i0 + ql_i) * block_bytes + (n0 >> 3) + (int64_t)row * row_bytes);
            }
            ql_i += 4;
            wrap_quad();
        };
        // the sign words of pair `sel` (0..3) of a quad, for every lane group
        auto sign_words = [&](const uint4_t &qd, int sel) {
            const int from = (16 * sel + lm) * 4;
            uint4_t r;
#pragma unroll
            for (int d = 0; d < 4; d++) r[d] = (uint32_t)__builtin_amdgcn_ds_bpermute(from, (int)qd[d]);
            return r;
        };
        quad[0] = quad[1] = (uint4_t){0, 0, 0, 0};
        request_quad(quad[0]);
#pragma unroll
        for (int k = 0; k < 3; k++) request_u(b_set[k]);

        // four blocks at a time, so that their loads are in flight together
        for (int q0 = 0; q0 < ib; q0 += 4) {
            half8_t v[4];
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const int i = min(q0 + k, ib - 1);
                v[k] = (half8_t){0, 0, 0, 0, 0, 0, 0, 0};
                if (sr < K) v[k] = *reinterpret_cast<const half8_t *>(vt + ((int64_t)i * K + sr) * N + n0 + 8 * sp);
            }
#pragma unroll
            for (int k = 0; k < 4; k++) {
                if (q0 + k < ib) {
#pragma unroll
                    for (int e = 0; e < 8; e++) vl[(q0 + k) * VBLOCK + (8 * sp + e) * VSTRIDE + sp * VGROUP_PAD + sr] = v[k][e];
                }
            }
        }
        if (PACKED && tid < SIGN_LUT_HALVES) lut[tid] = ((tid >> 2) >> (3 - (tid & 3))) & 1 ? (half_t)1.f : (half_t)-1.f;
        __syncthreads();

        // 16 rows per wave and step; the current pair is (rows m0.., block i)
        // The first block of a row step starts the sums (a product, not a sum with zero): cleared accumulators
        // would meet the running ones where the paths join, and the compiler then copies two dozen registers per block.
        float4_t acc[8];
        int i = 0, m0 = first_row;
        auto consume = [&](const half4_t &b_cur, const uint4_t &swc, auto first_tag) {
            constexpr bool FIRST = decltype(first_tag)::value;
            const int row = min(m0 + lm, M - 1);
            const half_t *vb = vl + i * VBLOCK + aoff;
            // all eight fragments first, and every product one patch ahead of the sign FMAs
            // that use it: neither the LDS nor the MFMA latency sits in front of them
            half4_t a[8];
#pragma unroll
            for (int s = 0; s < 8; s++)
                a[s] = *reinterpret_cast<const half4_t *>(vb + (32 * (s >> 1) + 4 * (s & 1)) * VSTRIDE + 4 * (s >> 1) * VGROUP_PAD);
            // the signs of a patch as four halves of +-1.0 from the table (16 entries of 8 bytes: one entry per
            // pair of banks, equal nibbles read the same address), multiplied in by a mixed-precision FMA
            half4_t sv[8];
            if (PACKED) {
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const uint32_t hi = ((swc[q] >> sh_hi) & 0x78u) | lut_base;
                    const uint32_t lo = (__builtin_amdgcn_alignbit(swc[q], swc[q], sh_lo) & 0x78u) | lut_base;
                    sv[2 * q] = *reinterpret_cast<lds_half4_ptr>(hi);
                    sv[2 * q + 1] = *reinterpret_cast<lds_half4_ptr>(lo);
                }
            }
            float4_t p_next = __builtin_amdgcn_mfma_f32_16x16x16f16(a[0], b_cur, (float4_t){0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
#pragma unroll
            for (int s = 0; s < 8; s++) {
                const float4_t p = p_next;
                if (s + 1 < 8)
                    p_next = __builtin_amdgcn_mfma_f32_16x16x16f16(a[s + 1], b_cur, (float4_t){0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
                if (PACKED) {
#pragma unroll
                    for (int j = 0; j < 4; j++) acc[s][j] = __builtin_fmaf(p[j], (float)sv[s][j], FIRST ? 0.f : acc[s][j]);   // (a plain product would not become a mixed-precision instruction)
                } else {
                    uint32_t t = *reinterpret_cast<const uint32_t *>(
                        sign + ((int64_t)(i0 + i) * M + row) * N + n0 + 32 * (s >> 1) + 8 * g + 4 * (s & 1));
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        uint32_t sf = ((t << (24 - 8 * j)) & 0x80000000u) | 0x3F800000u;
                        acc[s][j] = FIRST ? p[j] * __builtin_bit_cast(float, sf) : __builtin_fmaf(p[j], __builtin_bit_cast(float, sf), acc[s][j]);
                    }
                }
            }
            if (++i == ib) {
                if (m0 + lm < M) {
                    half_t *wp = w + (int64_t)(m0 + lm) * N + n0 + 8 * g;
#pragma unroll
                    for (int s = 0; s < 8; s += 2) {
                        half8_t o = {(half_t)acc[s][0], (half_t)acc[s][1], (half_t)acc[s][2], (half_t)acc[s][3],
                                     (half_t)acc[s + 1][0], (half_t)acc[s + 1][1], (half_t)acc[s + 1][2], (half_t)acc[s + 1][3]};
                        *reinterpret_cast<half8_t *>(wp + 16 * s) = o;      // 32 columns per pair of patches
                    }
                }
                i = 0;
                m0 += 64;
            }
        };
        const int n_pairs = first_row < row_end ? ((row_end - first_row + 63) / 64) * ib : 0;
        for (int p = 0; p < n_pairs; p += 8) {
#pragma unroll
            for (int idx = 0; idx < 8; idx++) {
                if (idx > 0 && p + idx >= n_pairs) break;
                const int h = idx >> 2, k = idx & 3;
                if (k == 0) request_quad(quad[h ^ 1]);          // the next quad, into the set consumed last
                request_u(b_set[(k + 3) & 3]);
                const uint4_t swc = sign_words(quad[h], k);
                if (i == 0)
                    consume(b_set[k], swc, std::true_type{});
                else
                    consume(b_set[k], swc, std::false_type{});
            }
        }
    }
}

// Any shape (also rows that do not start on a byte boundary): one output per
// thread, bit addressed through the flat element index.
template <bool PACKED>
__global__ __launch_bounds__(256) void reconstruct_generic_kernel(
    const uint8_t *__restrict__ packed, const int8_t *__restrict__ sign,
    const half_t *__restrict__ u, const half_t *__restrict__ vt, half_t *__restrict__ w,
    int I, int M, int N, int K) {
    const int64_t total = (int64_t)M * N;
    const int64_t block_bytes = (total + 7) >> 3;
    int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; e < total; e += stride) {
        const int m = (int)(e / N), n = (int)(e % N);
        float acc = 0.f;
        for (int i = 0; i < I; i++) {
            float p = 0.f;
            for (int r = 0; r < K; r++)
                p = __builtin_fmaf((float)u[((int64_t)i * M + m) * K + r],
                                   (float)vt[((int64_t)i * K + r) * N + n], p);
            float s;
            if (PACKED)
                s = ((packed[i * block_bytes + (e >> 3)] >> (7 - (int)(e & 7))) & 1) ? 1.f : -1.f;
            else
                s = (float)sign[(int64_t)i * total + e];
            acc += s * p;
        }
        w[e] = (half_t)acc;
    }
}

template <bool PACKED>
int launch_reconstruct(const uint8_t *packed, const int8_t *sign, const half_t *u, const half_t *vt,
                       half_t *w, int I, int M, int N, int K, hipStream_t s) {
    // the tiled kernel addresses a block's u and sign rows with 32-bit byte offsets
    const bool small = (int64_t)M * (N >> 3) < ((int64_t)1 << 32) && (int64_t)M * K * 2 < ((int64_t)1 << 32);
    const bool tiled = (N % RT_COLS == 0) && I >= 1 && I <= RT_MAXB && small && bs_aligned(vt, 16) && bs_aligned(w, 16) &&
                       bs_aligned(u, 8) && (PACKED ? bs_aligned(packed, 16) : bs_aligned(sign, 4));
    if (tiled) {
        // One wave of workgroups: as many row groups as the resident slots allow (LDS decides
        // how many workgroups a CU holds), so that no second, partial wave trails behind.
        // Every workgroup re-stages its vt strip, so rows per workgroup stay a multiple of 64.
        const int strips = N / RT_COLS, strips8 = (int)bs_cdiv(strips, 8) * 8;
        const size_t lds_need = (size_t)I * VBLOCK * sizeof(half_t) + SIGN_LUT_HALVES * sizeof(half_t);   // vt images + sign table
        int per_cu = (int)((160 * 1024) / lds_need);
        if (per_cu > 8) per_cu = 8;
        if (per_cu < 1) per_cu = 1;
        int row_groups = (256 * per_cu) / strips8;
        if (row_groups < 1) row_groups = 1;
        int rows_per_wg = (int)bs_cdiv(bs_cdiv(M, row_groups), 64) * 64;
        row_groups = (int)bs_cdiv(M, rows_per_wg);
        const size_t lds = lds_need;
        static bs_lds_grant granted[2][BS_MAX_DEVICES];
        const void *kernel = K == 16 ? (const void *)reconstruct_tile_kernel<PACKED, true> : (const void *)reconstruct_tile_kernel<PACKED, false>;
        const int st = bs_allow_lds(kernel, lds, granted[K == 16]);
        if (st != BS_OK) return st;
        dim3 grid((unsigned)bs_cdiv(strips, 8) * 8, row_groups);
        if (K == 16)
            reconstruct_tile_kernel<PACKED, true><<<grid, 256, lds, s>>>(packed, sign, u, vt, w, I, M, N, K, rows_per_wg);
        else
            reconstruct_tile_kernel<PACKED, false><<<grid, 256, lds, s>>>(packed, sign, u, vt, w, I, M, N, K, rows_per_wg);
    } else {
        int64_t blocks = bs_cdiv((int64_t)M * N, 256);
        if (blocks > 256 * 64) blocks = 256 * 64;
        reconstruct_generic_kernel<PACKED><<<(int)blocks, 256, 0, s>>>(packed, sign, u, vt, w, I, M, N, K);
    }
    BS_LAUNCH_CHECK();
    return BS_OK;
}

int check_dims(int I, int M, int N, int K) {
    if (I < 0 || M <= 0 || N <= 0) return BS_ERR_SHAPE;
    if (K < 1 || K > 16) return BS_ERR_RANK;
    if ((int64_t)M * N > ((int64_t)1 << 40)) return BS_ERR_SHAPE;
    return BS_OK;
}

}  // namespace

int bs_launch_reconstruct_packed(const uint8_t *packed, const half_t *u, const half_t *vt,
                                 half_t *w, int I, int M, int N, int K, hipStream_t s) {
    return launch_reconstruct<true>(packed, nullptr, u, vt, w, I, M, N, K, s);
}

extern "C" int bs_reconstruct_w(const uint8_t *packed, const void *u, const void *vt, void *w,
                                int I, int M, int N, int K, void *stream) {
    int st = check_dims(I, M, N, K);
    if (st != BS_OK) return st;
    if (!w || (I > 0 && (!packed || !u || !vt))) return BS_ERR_NULL;
    if (!bs_aligned(u, 2) || !bs_aligned(vt, 2) || !bs_aligned(w, 2)) return BS_ERR_ALIGN;
    return launch_reconstruct<true>(packed, nullptr, (const half_t *)u, (const half_t *)vt,
                                    (half_t *)w, I, M, N, K, (hipStream_t)stream);
}

extern "C" int bs_reconstruct_w_from_sign(const int8_t *sign, const void *u, const void *vt, void *w,
                                          int I, int M, int N, int K, void *stream) {
    int st = check_dims(I, M, N, K);
    if (st != BS_OK) return st;
    if (!w || (I > 0 && (!sign || !u || !vt))) return BS_ERR_NULL;
    if (!bs_aligned(u, 2) || !bs_aligned(vt, 2) || !bs_aligned(w, 2)) return BS_ERR_ALIGN;
    return launch_reconstruct<false>(nullptr, sign, (const half_t *)u, (const half_t *)vt,
                                     (half_t *)w, I, M, N, K, (hipStream_t)stream);
}

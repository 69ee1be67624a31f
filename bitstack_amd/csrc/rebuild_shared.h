// Pieces shared by the kernels that rebuild 16 x 16 patches of the weight in registers (strip.hip, panel.hip):
// the vt image of a strip in LDS, the sign table, and one block of a 16-row x 128-column patch row.
#pragma once

#include "common.h"

namespace {

constexpr int SF_COLS = 128;    // columns per strip
constexpr int VSTRIDE = 16;     // halves per column of the vt image: the 16 ranks
constexpr int VGROUP_PAD = 4;   // extra halves after every 8 columns
constexpr int VBLOCK = SF_COLS * VSTRIDE + (SF_COLS / 8) * VGROUP_PAD;   // halves per block
// The 16 sign nibbles as four halves each (+1.0 for a set bit, first column in the top bit), at the very start of
// LDS and 128-byte aligned: a nibble times 8, OR-ed into the table's address, is where its four signs lie.  16
// entries of 8 bytes take one pair of banks each and equal nibbles read the same address: no bank conflicts.
constexpr int SIGN_LUT_HALVES = 64;
typedef const __attribute__((address_space(3))) half4_t *lds_half4_ptr;
struct SignTable {
    uint32_t base;       // LDS address of the table
    int sh_hi, sh_lo;    // the lane's byte of a sign word is byte g: (word >> sh_hi) & 0x78 addresses the signs of its
                         // first four columns, (word rotated right by sh_lo) & 0x78 those of the other four
};
__device__ __forceinline__ SignTable make_sign_table(half_t *lut, int tid, int g) {
    if (tid < SIGN_LUT_HALVES) lut[tid] = ((tid >> 2) >> (3 - (tid & 3))) & 1 ? (half_t)1.f : (half_t)-1.f;
    SignTable st;
    st.base = (uint32_t)reinterpret_cast<uintptr_t>((const __attribute__((address_space(3))) half_t *)lut);
    st.sh_hi = 8 * g + 1;
    st.sh_lo = (8 * g - 3) & 31;
    return st;
}

// Register sets of (u rows, sign words) a wave's requests rotate through: they run NSETS - 1 (row step, strip,
// block) triples ahead.  The loops below are written out NSETS triples at a time, so that no set is ever copied
// into another: a copy waits for the load it copies, which would pull every request back to one triple ahead.
constexpr int NSETS = 3;

// One block of a 16-row x 128-column patch row: acc[s][j] += sign * (u . vt) for the eight 16 x 16 patches.
// vb: this lane's fragment of the block's vt image.  All eight fragments and all eight sign vectors are
// requested first, and every product runs one patch ahead of the FMAs that use it: neither the LDS nor the
// MFMA latency sits in front of them.
// FIRST: the sums start here (a zero addend; a plain product would not become a mixed-precision instruction).
template <bool FIRST>
__device__ __forceinline__ void rebuild_block(const half_t *vb, const half4_t b, const uint4_t sw, const SignTable st,
                                              float4_t (&acc)[8]) {
    half4_t a[8], sv[8];
#pragma unroll
    for (int s = 0; s < 8; s++)
        a[s] = *reinterpret_cast<const half4_t *>(vb + (32 * (s >> 1) + 4 * (s & 1)) * VSTRIDE + 4 * (s >> 1) * VGROUP_PAD);
    auto lookup = [&](int q) {      // the signs of patches 2q and 2q + 1
        const uint32_t hi = ((sw[q] >> st.sh_hi) & 0x78u) | st.base;
        const uint32_t lo = (__builtin_amdgcn_alignbit(sw[q], sw[q], st.sh_lo) & 0x78u) | st.base;
        sv[2 * q] = *reinterpret_cast<lds_half4_ptr>(hi);
        sv[2 * q + 1] = *reinterpret_cast<lds_half4_ptr>(lo);
    };
    lookup(0);
    float4_t p_next = __builtin_amdgcn_mfma_f32_16x16x16f16(a[0], b, (float4_t){0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
#pragma unroll
    for (int s = 0; s < 8; s++) {
        const float4_t p = p_next;
        if (s + 1 < 8) p_next = __builtin_amdgcn_mfma_f32_16x16x16f16(a[s + 1], b, (float4_t){0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
        if (s % 2 == 0 && s < 6) lookup(s / 2 + 1);   // the sign vectors of the next two patches, while these two are used
#pragma unroll
        for (int j = 0; j < 4; j++) acc[s][j] = __builtin_fmaf(p[j], (float)sv[s][j], FIRST ? 0.f : acc[s][j]);
    }
}

}  // namespace

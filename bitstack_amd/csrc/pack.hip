// Sign packing / unpacking for gfx950.
//
// Layout: flat element e lives in byte e / 8, bit 7 - e % 8; bit 1 = +1.
// Both kernels are pure streaming (unpack writes eight bytes per byte read),
// so the only concerns are wide coalesced accesses and enough workgroups.
#include "common.h"

namespace {

// Four packed bytes -> 32 int8 signs, written as two 16-byte stores.
// After a full bit reversal of the little-endian word, byte 3-b holds source
// byte b with element j of that byte in bit j, so a multiply spreads a nibble
// over four byte lanes in element order.
__device__ inline uint32_t spread_nibble(uint32_t nib) {
    uint32_t ones = (nib * 0x00204081u) & 0x01010101u;        // byte j = bit j of nib
    return 0x01010101u | ((ones ^ 0x01010101u) * 0xFEu);      // 1 -> 0x01, 0 -> 0xFF
}

__global__ __launch_bounds__(256) void unpack_words_kernel(const uint32_t *__restrict__ packed,
                                                           uint4_t *__restrict__ out,
                                                           int64_t n_words) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < n_words; i += stride) {
        uint32_t r = __builtin_bitreverse32(packed[i]);
        uint4_t lo, hi;
        // source byte 0 sits in bits 31..24 of r, byte 3 in bits 7..0
        lo.x = spread_nibble((r >> 24) & 0xF);
        lo.y = spread_nibble((r >> 28) & 0xF);
        lo.z = spread_nibble((r >> 16) & 0xF);
        lo.w = spread_nibble((r >> 20) & 0xF);
        hi.x = spread_nibble((r >> 8) & 0xF);
        hi.y = spread_nibble((r >> 12) & 0xF);
        hi.z = spread_nibble(r & 0xF);
        hi.w = spread_nibble((r >> 4) & 0xF);
        out[2 * i] = lo;
        out[2 * i + 1] = hi;
    }
}

// Any alignment, any length: one element per thread.
__global__ __launch_bounds__(256) void unpack_elems_kernel(const uint8_t *__restrict__ packed,
                                                           int8_t *__restrict__ out,
                                                           int64_t first, int64_t n_elems) {
    int64_t e = first + (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; e < n_elems; e += stride) {
        int bit = (packed[e >> 3] >> (7 - (int)(e & 7))) & 1;
        out[e] = (int8_t)(2 * bit - 1);
    }
}

// One output byte per thread; eight int8 reads (one 8-byte load when aligned).
__global__ __launch_bounds__(256) void pack_kernel(const int8_t *__restrict__ sign,
                                                   uint8_t *__restrict__ packed,
                                                   int64_t n_elems, int aligned8) {
    int64_t nbytes = (n_elems + 7) >> 3;
    int64_t j = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; j < nbytes; j += stride) {
        uint32_t b = 0;
        if (aligned8 && 8 * j + 8 <= n_elems) {
            uint64_t v = *reinterpret_cast<const uint64_t *>(sign + 8 * j);
#pragma unroll
            for (int i = 0; i < 8; i++) {
                int8_t s = (int8_t)(v >> (8 * i));
                b |= (uint32_t)(s > 0) << (7 - i);
            }
        } else {
            for (int i = 0; i < 8; i++) {
                int64_t e = 8 * j + i;
                if (e < n_elems) b |= (uint32_t)(sign[e] > 0) << (7 - i);
            }
        }
        packed[j] = (uint8_t)b;
    }
}

inline int grid_for(int64_t items, int block) {
    int64_t g = bs_cdiv(items, block);
    const int64_t cap = 256 * 32;   // 32 workgroups per CU is plenty for a streaming kernel
    return (int)(g < 1 ? 1 : (g > cap ? cap : g));
}

}  // namespace

extern "C" int bs_unpack_sign(const uint8_t *packed, int8_t *out, int64_t n_elems, void *stream) {
    if (n_elems < 0) return BS_ERR_SHAPE;
    if (n_elems == 0) return BS_OK;
    if (!packed || !out) return BS_ERR_NULL;
    hipStream_t s = (hipStream_t)stream;
    int64_t done = 0;
    if (bs_aligned(packed, 4) && bs_aligned(out, 16)) {
        int64_t n_words = n_elems / 32;
        if (n_words > 0) {
            unpack_words_kernel<<<grid_for(n_words, 256), 256, 0, s>>>(
                reinterpret_cast<const uint32_t *>(packed), reinterpret_cast<uint4_t *>(out), n_words);
            BS_LAUNCH_CHECK();
            done = n_words * 32;
        }
    }
    if (done < n_elems) {
        unpack_elems_kernel<<<grid_for(n_elems - done, 256), 256, 0, s>>>(packed, out, done, n_elems);
        BS_LAUNCH_CHECK();
    }
    return BS_OK;
}

extern "C" int bs_pack_sign(const int8_t *sign, uint8_t *packed, int64_t n_elems, void *stream) {
    if (n_elems < 0) return BS_ERR_SHAPE;
    if (n_elems == 0) return BS_OK;
    if (!sign || !packed) return BS_ERR_NULL;
    int64_t nbytes = (n_elems + 7) / 8;
    pack_kernel<<<grid_for(nbytes, 256), 256, 0, (hipStream_t)stream>>>(sign, packed, n_elems,
                                                                      bs_aligned(sign, 8) ? 1 : 0);
    BS_LAUNCH_CHECK();
    return BS_OK;
}

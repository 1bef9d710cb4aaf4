// Bitplane layout helpers and the in-lane plane -> index transpose.
//
// Everything here is pure integer code that compiles for the GPU (hipcc) and
// for the host (g++, used by the CPU unit tests of these bit tricks).
//
// Packed layout (reference: any_precision/quantization/pack.py:12-76,90-99,
// consumed at any_precision/modules/kernels/dequant.cuh:215-240): qweight is
// uint32 [planes, N, K/32]; plane 0 is the MSB of the parent code.  A row is
// cut into chunks of 32 words (1024 elements); the last chunk may hold only
// T = (K % 1024) / 32 words.  Word t of chunk c, byte b (b = 0 is the low
// byte), bit u of that byte holds element
//     k = 1024 c + 8 (T (3 - b) + t) + (7 - u).
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define AP_HD __host__ __device__ __forceinline__
#else
#define AP_HD inline
#endif

namespace ap {

// Words in the chunk that contains word `w` of a row of K elements.
AP_HD int chunk_words(int w, int K) {
    return ((w >> 5) == (K >> 10)) ? ((K & 1023) >> 5) : 32;
}

// First element (of 8 consecutive ones) that byte-group j = 3 - b of word w covers.
AP_HD int group_base(int w, int j, int K) {
    const int c = w >> 5, t = w & 31;
    return (c << 10) + 8 * (chunk_words(w, K) * j + t);
}

// One butterfly step of an 8x8 bit-matrix transpose carried out in the four
// byte columns of a word at once: exchanges the S-bit blocks selected by
// `lo_mask` between word a (keeps its low blocks) and word b (keeps its high).
template <int S, uint32_t LO>
AP_HD void swap_blocks(uint32_t &a, uint32_t &b) {
    const uint32_t na = (a & LO) | ((b << S) & ~LO);
    const uint32_t nb = ((a >> S) & LO) | (b & ~LO);
    a = na;
    b = nb;
}

// q[p], p = 0..BITS-1: the word of plane p (plane 0 most significant) for 32
// elements.  idx[e], e = 0..7: byte b of idx[e] is the BITS-bit index of the
// element stored at bit 8 b + (7 - e) of the plane words, shifted left by
// SHIFT (SHIFT + BITS <= 8).  Same result as the reference's
// dequant<bits,false> (dequant.cuh:32-175) when SHIFT = 0, reached with a
// three-stage butterfly (48 bit-ops for 8 planes instead of 8 x 22).
template <int BITS, int SHIFT = 0>
AP_HD void planes_to_indices(const uint32_t (&q)[BITS], uint32_t (&idx)[8]) {
    static_assert(BITS >= 1 && BITS + SHIFT <= 8, "index must fit a byte");
    uint32_t r[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        // bit i of the output byte comes from row i: plane BITS-1-(i-SHIFT)
        const int p = BITS - 1 - (i - SHIFT);
        r[i] = (p >= 0 && p < BITS) ? q[p >= 0 && p < BITS ? p : 0] : 0u;
    }
#pragma unroll
    for (int i = 0; i < 4; i++) swap_blocks<4, 0x0F0F0F0Fu>(r[i], r[i + 4]);
#pragma unroll
    for (int i = 0; i < 8; i += 4) {
        swap_blocks<2, 0x33333333u>(r[i], r[i + 2]);
        swap_blocks<2, 0x33333333u>(r[i + 1], r[i + 3]);
    }
#pragma unroll
    for (int i = 0; i < 8; i += 2) swap_blocks<1, 0x55555555u>(r[i], r[i + 1]);
    // r[u] byte b bit i = row i bit (8 b + u); element e sits at u = 7 - e.
#pragma unroll
    for (int e = 0; e < 8; e++) idx[e] = r[7 - e];
}

// Pair form (reference: dequant<3,true>, dequant<4,true>, dequant.cuh:13-30,
// 56-67): byte b of pidx[m], m = 0..3, is (index(e = m) << BITS) | index(e = m + 4).
template <int BITS>
AP_HD void planes_to_pair_indices(const uint32_t (&q)[BITS], uint32_t (&pidx)[4]) {
    static_assert(BITS <= 4, "pair index must fit a byte");
    uint32_t idx[8];
    planes_to_indices<BITS, 0>(q, idx);
#pragma unroll
    for (int m = 0; m < 4; m++) pidx[m] = (idx[m] << BITS) | idx[m + 4];
}

}  // namespace ap

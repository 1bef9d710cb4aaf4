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
#include <hip/hip_runtime.h>
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

// (a & mask) | (b & ~mask): one v_bitop3_b32 on the GPU.
AP_HD uint32_t bit_select(uint32_t mask, uint32_t a, uint32_t b) {
#if defined(__HIP_DEVICE_COMPILE__)
    return __builtin_amdgcn_bitop3_b32(a, b, mask, 0xE4);
#else
    return (a & mask) | (b & ~mask);
#endif
}

// One butterfly step of a bit-matrix transpose carried out in every byte (or
// nibble) of a word at once: exchanges the S-bit blocks selected by LO
// between word a (keeps its low blocks) and word b (keeps its high blocks).
// Each output is one shift and one three-input bitwise select; AZERO / BZERO
// say that a / b is known to be zero, which saves the select.
template <int S, uint32_t LO, bool AZERO = false, bool BZERO = false>
AP_HD void swap_blocks(uint32_t &a, uint32_t &b) {
    uint32_t na, nb;
    if constexpr (AZERO && BZERO) {
        na = 0u;
        nb = 0u;
    } else if constexpr (BZERO) {
        na = a & LO;
        nb = (a >> S) & LO;
    } else if constexpr (AZERO) {
        na = (b << S) & ~LO;
        nb = b & ~LO;
    } else {
        na = bit_select(LO, a, b << S);
        nb = bit_select(LO, a >> S, b);
    }
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
    // row i feeds bit i of the output byte: plane BITS-1-(i-SHIFT), zero outside
    constexpr int LOW = SHIFT, HIGH = SHIFT + BITS;   // rows [LOW, HIGH) are live
#define AP_LIVE(i) ((i) >= LOW && (i) < HIGH)
    uint32_t r[8];
#pragma unroll
    for (int i = 0; i < 8; i++) r[i] = AP_LIVE(i) ? q[AP_LIVE(i) ? BITS - 1 - (i - SHIFT) : 0] : 0u;
    // stage 1: 4-bit blocks between rows i and i+4
    swap_blocks<4, 0x0F0F0F0Fu, !AP_LIVE(0), !AP_LIVE(4)>(r[0], r[4]);
    swap_blocks<4, 0x0F0F0F0Fu, !AP_LIVE(1), !AP_LIVE(5)>(r[1], r[5]);
    swap_blocks<4, 0x0F0F0F0Fu, !AP_LIVE(2), !AP_LIVE(6)>(r[2], r[6]);
    swap_blocks<4, 0x0F0F0F0Fu, !AP_LIVE(3), !AP_LIVE(7)>(r[3], r[7]);
    // after stage 1 rows i and i+4 are live iff either was
#define AP_LIVE1(i) (AP_LIVE((i) & 3) || AP_LIVE(((i) & 3) + 4))
    swap_blocks<2, 0x33333333u, !AP_LIVE1(0), !AP_LIVE1(2)>(r[0], r[2]);
    swap_blocks<2, 0x33333333u, !AP_LIVE1(1), !AP_LIVE1(3)>(r[1], r[3]);
    swap_blocks<2, 0x33333333u, !AP_LIVE1(4), !AP_LIVE1(6)>(r[4], r[6]);
    swap_blocks<2, 0x33333333u, !AP_LIVE1(5), !AP_LIVE1(7)>(r[5], r[7]);
#define AP_LIVE2(i) (AP_LIVE1((i) & 5) || AP_LIVE1(((i) & 5) + 2))
    swap_blocks<1, 0x55555555u, !AP_LIVE2(0), !AP_LIVE2(1)>(r[0], r[1]);
    swap_blocks<1, 0x55555555u, !AP_LIVE2(2), !AP_LIVE2(3)>(r[2], r[3]);
    swap_blocks<1, 0x55555555u, !AP_LIVE2(4), !AP_LIVE2(5)>(r[4], r[5]);
    swap_blocks<1, 0x55555555u, !AP_LIVE2(6), !AP_LIVE2(7)>(r[6], r[7]);
#undef AP_LIVE2
#undef AP_LIVE1
#undef AP_LIVE
    // r[u] byte b bit i = row i bit (8 b + u); element e sits at u = 7 - e.
#pragma unroll
    for (int e = 0; e < 8; e++) idx[e] = r[7 - e];
}

// Adjacent-pair form for BITS = 3, 4: apair[i], i = 0..3; byte b of apair[i] addresses the table entry
// of the element PAIR (2i, 2i+1) of byte group 3 - b -- two elements that also share a dword of the
// fp16 activations, so the activations need no rearranging (the reference's dequant<3,true> and
// dequant<4,true>, dequant.cuh:13-30,56-67, pair element e with e + 4).
// The byte holds the two indices bit-interleaved: with A = index(2i), B = index(2i+1) and A_k the bit
// of weight 2^k,
//     BITS = 4:  byte = A3 B3 A2 B2 A1 B1 A0 B0                       (entry number of a 256-entry table)
//     BITS = 3:  byte = A2 B2 A1 B1 A0 B0 0 0                         (BYTE OFFSET into 64 dword entries)
// Built as a 4 x 4 transpose of the 2-bit blocks of every byte across the plane words: two butterfly
// stages, 16 bit-ops for 4 planes and 14 for 3 (one row is zero).
template <int BITS>
AP_HD void planes_to_adjacent_pairs(const uint32_t (&q)[BITS], uint32_t (&apair)[4]) {
    static_assert(BITS == 3 || BITS == 4, "pair tables exist for 3 and 4 bits");
    // row k supplies block k of the output byte: the plane of weight 2^k (BITS = 4), or of weight 2^(k-1)
    // with a zero row 0 (BITS = 3)
    uint32_t r[4];
    constexpr bool Z0 = BITS == 3;
    r[0] = Z0 ? 0u : q[3];
    r[1] = q[BITS - 1 - (Z0 ? 0 : 1)];
    r[2] = q[BITS - 2 - (Z0 ? 0 : 1)];
    r[3] = q[0];
    swap_blocks<4, 0x0F0F0F0Fu, Z0, false>(r[0], r[2]);
    swap_blocks<4, 0x0F0F0F0Fu>(r[1], r[3]);
    swap_blocks<2, 0x33333333u>(r[0], r[1]);
    swap_blocks<2, 0x33333333u>(r[2], r[3]);
    // r[m] collects block m (bits 2m+1, 2m = elements 6-2m, 7-2m) of every plane: pair i = 3 - m
#pragma unroll
    for (int i = 0; i < 4; i++) apair[i] = r[3 - i];
}

// The two table indices a byte of planes_to_adjacent_pairs stands for (host and device; the kernels use
// it to build their pair tables): first = index of element 2i, second = index of element 2i+1.
template <int BITS>
AP_HD void adjacent_pair_split(uint32_t byte, uint32_t &first, uint32_t &second) {
    const uint32_t v = BITS == 3 ? byte >> 2 : byte;
    first = ((v >> 1) & 1u) | ((v >> 2) & 2u) | ((v >> 3) & 4u) | ((v >> 4) & 8u);
    second = (v & 1u) | ((v >> 1) & 2u) | ((v >> 2) & 4u) | ((v >> 3) & 8u);
}

}  // namespace ap

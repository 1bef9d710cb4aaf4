// Host build of the pure-integer device helpers, for the CPU unit tests.
// Compiled with g++ into libanyprec_hostcheck.so; exports the in-lane plane ->
// index transposes and the layout address helpers exactly as the kernels use them.
#include "ap_bitplane.hpp"
#include "ap_reciprocal.hpp"

extern "C" {

int aph_planes_to_indices(const uint32_t *q, int bits, int shift, uint32_t *idx) {
    uint32_t out[8];
#define AP_CASE(B, S)                                        \
    if (bits == B && shift == S) {                           \
        uint32_t qq[B];                                      \
        for (int i = 0; i < B; i++) qq[i] = q[i];            \
        ap::planes_to_indices<B, S>(qq, out);                \
        for (int i = 0; i < 8; i++) idx[i] = out[i];         \
        return 0;                                            \
    }
    AP_CASE(1, 0) AP_CASE(2, 0) AP_CASE(3, 0) AP_CASE(4, 0) AP_CASE(5, 0) AP_CASE(6, 0) AP_CASE(7, 0) AP_CASE(8, 0)
    AP_CASE(3, 1) AP_CASE(4, 1) AP_CASE(5, 1) AP_CASE(6, 1) AP_CASE(7, 1)
#undef AP_CASE
    return -1;
}

int aph_planes_to_adjacent_pairs(const uint32_t *q, int bits, uint32_t *apair) {
    uint32_t out[4];
    if (bits == 3) {
        uint32_t qq[3] = {q[0], q[1], q[2]};
        ap::planes_to_adjacent_pairs<3>(qq, out);
    } else if (bits == 4) {
        uint32_t qq[4] = {q[0], q[1], q[2], q[3]};
        ap::planes_to_adjacent_pairs<4>(qq, out);
    } else {
        return -1;
    }
    for (int i = 0; i < 4; i++) apair[i] = out[i];
    return 0;
}

int aph_adjacent_pair_split(int bits, uint32_t byte, uint32_t *first, uint32_t *second) {
    if (bits == 3) ap::adjacent_pair_split<3>(byte, *first, *second);
    else if (bits == 4) ap::adjacent_pair_split<4>(byte, *first, *second);
    else return -1;
    return 0;
}

int aph_chunk_words(int w, int K) { return ap::chunk_words(w, K); }
int aph_group_base(int w, int j, int K) { return ap::group_base(w, j, K); }

// n / d and n % d through the host-side reciprocal, as the dequantiser numbers its segments (n < 2^31)
int aph_divmod_by_reciprocal(uint32_t n, uint32_t d, uint32_t *q, uint32_t *r) {
    if (d < 1 || d >= (1u << 31) || n >= (1u << 31)) return -1;
    ap::divmod_by_reciprocal(n, d, ap::reciprocal_floor(d), *q, *r);
    return 0;
}

// n / d as the K-split GEMM splits its steps over d waves (n * d < 2^32)
int aph_div_by_reciprocal_ceil(uint32_t n, uint32_t d, uint32_t *q) {
    if (d < 1 || (unsigned long long)n * d >= (1ull << 32)) return -1;
    *q = ap::div_by_reciprocal_ceil(n, d, ap::reciprocal_ceil(d));
    return 0;
}

}  // extern "C"

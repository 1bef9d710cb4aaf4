// Fine-grained bitplane GEMV for gfx950, 1 <= M <= 4, rows of a multiple of 64 elements:
//     out[m,n] = sum_k x[m,k] * lut[n, index_b(n,k)]      (fp32 accumulate, fp16 out)
//
// Same contract as the reference's matmul_kbit_32 (any_precision/modules/kernels/matmul.cuh:16-167).
// One workgroup per ROW PAIR, one wave per 64 words (2048 elements) of the pair, one word of either row
// per lane: the launch is many short waves, so the waves whose planes arrive first compute while the
// rest of the matrix is still streaming in.  What a wave does besides its lookups is kept minimal:
//   * planes: one 8-byte load per plane -- lanes 0..31 take words 2l, 2l+1 of the even row, lanes
//     32..63 the same words of the odd row (512 contiguous bytes per row) -- and one v_permlane32_swap
//     per plane hands every lane word 2(l%32) + l/32 of BOTH rows, so the 16 activation registers of
//     that word serve two rows and the two tables sit at compile-time LDS addresses;
//   * activations: four 16-byte loads, used as they are (the pair tables of 3 and 4 bits pair adjacent
//     elements, ap_lookup.hpp);
//   * the S segment sums of a row meet in LDS and are added in wave order (deterministic).
#pragma once
#include "ap_gemvf_launch.hpp"
#include "ap_lookup.hpp"

namespace ap {

constexpr int kGemvfSegWords = 64;  // words of a row one wave covers

// Grid: N / 2 workgroups of (64, S) threads, S = ceil(K / 2048) <= THREADS / 64.  N even, K a multiple of
// 64, out 4-byte aligned.
template <int BITS, int M, int THREADS>
__global__ __launch_bounds__(THREADS) void gemvf_kbit_kernel(const half_t *__restrict__ x,
                                                            const uint32_t *__restrict__ qweight,
                                                            const half_t *__restrict__ lut, half_t *__restrict__ out,
                                                            int N, int K) {
    constexpr int NC = 1 << BITS;
    constexpr bool kMulti = THREADS > kWave;
    constexpr int MAXS = THREADS / kWave;
    __shared__ __attribute__((aligned(16))) uint8_t tables[2][LookupTable<BITS>::kBytes];
    __shared__ float partial[MAXS][2 * M];

    const int lane = threadIdx.x;
    const int s = kMulti ? __builtin_amdgcn_readfirstlane(threadIdx.y) : 0;
    const int S = kMulti ? (int)blockDim.y : 1;
    const int W = K >> 5;
    const size_t plane_stride = (size_t)N * W;
    const int pair = blockIdx.x;

    const uint32_t half = (uint32_t)lane >> 5, l5 = (uint32_t)lane & 31u;
    const uint32_t seg_word = (uint32_t)s * kGemvfSegWords + 2u * l5;  // first word of this lane's 8-byte load
    const bool valid = seg_word < (uint32_t)W;                         // lanes past the row end idle (sums dropped)
    const uint32_t lane_off = half * (uint32_t)W + (valid ? seg_word : 0u);
    const uint32_t w0 = valid ? seg_word + half : 0u;                  // this lane's word after the regroup

    // issue order: tables (tiny, staged while the planes are in flight), planes (HBM), activations (L2)
    const PairLane<BITS> pl = pair_lane<BITS>(lane);
    TableWords<BITS> t[2];
#pragma unroll
    for (int r = 0; r < 2; r++)
        if (s == r % S) t[r] = lookup_table_fetch<BITS>(lut + (size_t)(2 * pair + r) * NC, lane, pl);
    u32x2 q[BITS];
    const uint32_t *row_base = qweight + (size_t)(2 * pair) * W;
#pragma unroll
    for (int p = 0; p < BITS; p++)  // streamed once: non-temporal, so x and the tables keep their cache lines
        q[p] = load_at_nt<u32x2>(scalar_ptr(row_base + p * plane_stride), lane_off * (uint32_t)sizeof(uint32_t));
    uint32_t X[M][1][4][4];
    load_activations_plain<M, 1>(x, K, (int)w0, X);
#pragma unroll
    for (int r = 0; r < 2; r++)
        if (s == r % S) {
            lookup_table_arrive<BITS>(t[r]);  // staging arithmetic stays behind the plane and activation loads
            lookup_table_stage<BITS>(t[r], tables[r], lane);
        }
    if constexpr (kMulti) lds_only_barrier(); else __builtin_amdgcn_wave_barrier();

    uint32_t words[2][BITS];  // [row of the pair][plane]
#pragma unroll
    for (int p = 0; p < BITS; p++) {
        const auto a = __builtin_amdgcn_permlane32_swap(q[p][0], q[p][1], false, false);
        words[0][p] = a[0];
        words[1][p] = a[1];
    }
    float acc[2][M][2];
#pragma unroll
    for (int r = 0; r < 2; r++)
#pragma unroll
        for (int m = 0; m < M; m++) acc[r][m][0] = acc[r][m][1] = 0.f;
    lookup_dot<BITS, M, 2, 2, 1>(words, tables, X, acc, [](auto n) { return n; },
                                 [](auto) { return std::integral_constant<int, 0>{}; });
    float tot[2][M];
#pragma unroll
    for (int r = 0; r < 2; r++)
#pragma unroll
        for (int m = 0; m < M; m++) {
            float v = acc[r][m][0] + acc[r][m][1];
            asm volatile("" : "+v"(v));  // keeps the lookup stream out of an "if (valid)" region
            tot[r][m] = wave_sum(valid ? v : 0.f);
        }

    // fp16 results of rows 2*pair and 2*pair + 1 side by side: one 4-byte store per activation row
    auto store_pair = [&](int m, float even_sum, float odd_sum) {
        const half2_t v = {(half_t)even_sum, (half_t)odd_sum};
        *reinterpret_cast<half2_t *>(out + (size_t)m * N + 2 * pair) = v;
    };
    if constexpr (!kMulti) {
        if (lane == kSumLane) {
#pragma unroll
            for (int m = 0; m < M; m++) store_pair(m, tot[0][m], tot[1][m]);
        }
    } else {
        if (lane == kSumLane) {
#pragma unroll
            for (int r = 0; r < 2; r++)
#pragma unroll
                for (int m = 0; m < M; m++) partial[s][r * M + m] = tot[r][m];
        }
        lds_only_barrier();
        if (s == 0 && lane < M) {
            float even_sum = 0.f, odd_sum = 0.f;
            for (int ss = 0; ss < S; ss++) {
                even_sum += partial[ss][lane];
                odd_sum += partial[ss][M + lane];
            }
            store_pair(lane, even_sum, odd_sum);
        }
    }
}

}  // namespace ap

// Row-streaming bitplane GEMV for gfx950, 1 <= M <= 4, rows of a multiple of 128 elements:
//     out[m,n] = sum_k x[m,k] * lut[n, index_b(n,k)]      (fp32 accumulate, fp16 out)
//
// Same result as gemv_kbit_kernel (ap_gemv.hpp) and the same reference kernel
// (any_precision/modules/kernels/matmul.cuh:16-167), built for long-lived waves:
//   * A workgroup is the S waves that cover one row (wave s owns the 128 words = 4096
//     elements of K-segment s) and walks row PAIRS pair = blockIdx.x, + gridDim.x, ...: the
//     activations a lane needs never change, so they are loaded into registers once per wave
//     and the loads of the next pair are in flight while the current one is computed.
//   * Plane words are fetched with 16-byte loads: lanes 0..31 take words 4l..4l+3 of the
//     even row of the pair and lanes 32..63 the same words of the odd row, so with rows of
//     4096 elements one instruction reads 1 KB of contiguous memory.  Two v_permlane32_swap
//     per plane then hand every lane two words of BOTH rows (lane l: words 4(l%32) + 2(l/32)
//     and the next one): the whole wave works on one row at a time, every table sits at a
//     compile-time LDS address and a lookup address is a single instruction (ap_lookup.hpp).
//   * With S = 1 a workgroup is a single wave: no barrier anywhere; the tables of the next
//     pair overwrite those of the current one in place, because the LDS executes the
//     operations of one wave in order.  With S > 1 two LDS-only barriers per pair order the
//     tables and the exchange of the segment sums, which are added in wave order
//     (deterministic).
#pragma once
#include "ap_gemvp_launch.hpp"
#include "ap_lookup.hpp"

namespace ap {

constexpr int kGemvpSegWords = 128;  // words of a row one wave covers

// The planes of one row pair as they arrive: v[p] = words 4l..4l+3 of plane p, even row in
// lanes 0..31, odd row in lanes 32..63.
template <int BITS>
struct PairPlanes {
    u32x4 v[BITS];
};

template <int BITS>
__device__ __forceinline__ void load_pair(PairPlanes<BITS> &q, const uint32_t *__restrict__ row_base,
                                          size_t plane_stride, uint32_t lane_off) {
#pragma unroll
    for (int p = 0; p < BITS; p++)  // streamed once: non-temporal, so x and the tables keep their cache lines
        q.v[p] = load_at_nt<u32x4>(scalar_ptr(row_base + p * plane_stride), lane_off * (uint32_t)sizeof(uint32_t));
}

// Grid: G workgroups of (64, S) threads, S = ceil(K / 4096) <= THREADS / 64; workgroup g takes the row
// pairs g, g + G, ...  N even, K a multiple of 128, out 4-byte aligned.
template <int BITS, int M, int THREADS>
__global__ __launch_bounds__(THREADS) void gemvp_kbit_kernel(const half_t *__restrict__ x,
                                                            const uint32_t *__restrict__ qweight,
                                                            const half_t *__restrict__ lut, half_t *__restrict__ out,
                                                            int N, int K) {
    constexpr int NC = 1 << BITS;
    constexpr bool kMulti = THREADS > kWave;
    constexpr int MAXS = THREADS / kWave;
    constexpr int NBUF = 1;
    __shared__ __attribute__((aligned(16))) uint8_t tables[NBUF][2][LookupTable<BITS>::kBytes];
    __shared__ float partial[NBUF][MAXS][2 * M];

    const int lane = threadIdx.x;
    const int s = kMulti ? __builtin_amdgcn_readfirstlane(threadIdx.y) : 0;
    const int S = kMulti ? (int)blockDim.y : 1;
    const int W = K >> 5;
    const size_t plane_stride = (size_t)N * W;
    const int pairs = N >> 1, G = gridDim.x;

    const uint32_t half = (uint32_t)lane >> 5, l5 = (uint32_t)lane & 31u;
    const uint32_t seg_word = (uint32_t)s * kGemvpSegWords + 4u * l5;  // first word of this lane's 16-byte load
    const bool valid = seg_word < (uint32_t)W;                         // lanes past the row end idle (sums dropped)
    const uint32_t lane_off = half * (uint32_t)W + (valid ? seg_word : 0u);
    const uint32_t w0 = valid ? seg_word + 2u * half : 0u;             // this lane's two words after the regroup

    const PairLane<BITS> pl = pair_lane<BITS>(lane);
    auto fetch_tables = [&](int pair, TableWords<BITS>(&t)[2]) {
#pragma unroll
        for (int r = 0; r < 2; r++)
            if (s == r % S) t[r] = lookup_table_fetch<BITS>(lut + (size_t)(2 * pair + r) * NC, lane, pl);
    };
    auto stage_tables = [&](TableWords<BITS>(&t)[2], uint8_t(&slot)[2][LookupTable<BITS>::kBytes]) {
#pragma unroll
        for (int r = 0; r < 2; r++)
            if (s == r % S) {
                lookup_table_arrive<BITS>(t[r]);  // staging arithmetic stays behind the loads issued since the fetch
                lookup_table_stage<BITS>(t[r], slot[r], lane);
            }
    };

    int pair = blockIdx.x;  // the grid never exceeds the number of pairs
    PairPlanes<BITS> q, qn;
    TableWords<BITS> t[2], tn[2];
    fetch_tables(pair, t);
    load_pair<BITS>(q, qweight + (size_t)(2 * pair) * W, plane_stride, lane_off);
    uint32_t X[M][2][4][4];
    load_activations_plain<M, 2>(x, K, (int)w0, X);
    stage_tables(t, tables[0]);

    // One pair: sums of the even and the odd row over this wave's segment, valid in lane kSumLane.
    auto compute = [&](const PairPlanes<BITS> &planes, const uint8_t(&slot)[2][LookupTable<BITS>::kBytes],
                       float(&tot)[2][M]) {
        // word n of the stream = word n % 2 of row n / 2
        uint32_t words[4][BITS];
#pragma unroll
        for (int p = 0; p < BITS; p++) {
            const auto a = __builtin_amdgcn_permlane32_swap(planes.v[p][0], planes.v[p][2], false, false);
            const auto b = __builtin_amdgcn_permlane32_swap(planes.v[p][1], planes.v[p][3], false, false);
            words[0][p] = a[0];
            words[1][p] = b[0];
            words[2][p] = a[1];
            words[3][p] = b[1];
        }
        float acc[2][M][2];
#pragma unroll
        for (int r = 0; r < 2; r++)
#pragma unroll
            for (int m = 0; m < M; m++) acc[r][m][0] = acc[r][m][1] = 0.f;
        lookup_dot<BITS, M, 4, 2, 2>(words, slot, X, acc,
                                     [](auto n) { return std::integral_constant<int, decltype(n)::value / 2>{}; },
                                     [](auto n) { return std::integral_constant<int, decltype(n)::value % 2>{}; });
#pragma unroll
        for (int r = 0; r < 2; r++)
#pragma unroll
            for (int m = 0; m < M; m++) {
                float v = acc[r][m][0] + acc[r][m][1];
                // opaque to the optimiser: otherwise it moves the whole dot-product stream under
                // "if (valid)", behind all of its LDS reads, and the pipelining above is gone
                asm volatile("" : "+v"(v));
                tot[r][m] = wave_sum(valid ? v : 0.f);
            }
    };
    // fp16 results of rows 2*pair and 2*pair + 1 side by side: one 4-byte store per activation row
    auto store_pair = [&](int pr, int m, float even_sum, float odd_sum) {
        const half2_t v = {(half_t)even_sum, (half_t)odd_sum};
        *reinterpret_cast<half2_t *>(out + (size_t)m * N + 2 * pr) = v;
    };

    // Loop shape: every iteration but the last issues the loads of the pair after it before it
    // computes; the last one is peeled, so that no iteration waits on a path-merged load counter.
    if constexpr (!kMulti) {
        while (pair + G < pairs) {
            const int next = pair + G;
            fetch_tables(next, tn);
            load_pair<BITS>(qn, qweight + (size_t)(2 * next) * W, plane_stride, lane_off);
            __builtin_amdgcn_wave_barrier();
            float tot[2][M];
            compute(q, tables[0], tot);
            if (lane == kSumLane) {
#pragma unroll
                for (int m = 0; m < M; m++) store_pair(pair, m, tot[0][m], tot[1][m]);
            }
            // in-order LDS: these writes execute after the gathers of the pair just computed
            stage_tables(tn, tables[0]);
            q = qn;
            pair = next;
        }
        __builtin_amdgcn_wave_barrier();
        float tot[2][M];
        compute(q, tables[0], tot);
        if (lane == kSumLane) {
#pragma unroll
            for (int m = 0; m < M; m++) store_pair(pair, m, tot[0][m], tot[1][m]);
        }
    } else {
        // sums of this wave's segment -> LDS; after the barrier wave 0 adds the segments in order
        auto publish = [&](const float(&tot)[2][M]) {
            if (lane == kSumLane) {
#pragma unroll
                for (int r = 0; r < 2; r++)
#pragma unroll
                    for (int m = 0; m < M; m++) partial[0][s][r * M + m] = tot[r][m];
            }
        };
        auto combine = [&](int pr) {
            if (s == 0 && lane < M) {
                float even_sum = 0.f, odd_sum = 0.f;
                for (int ss = 0; ss < S; ss++) {
                    even_sum += partial[0][ss][lane];
                    odd_sum += partial[0][ss][M + lane];
                }
                store_pair(pr, lane, even_sum, odd_sum);
            }
        };
        lds_only_barrier();  // tables of the first pair staged
        while (pair + G < pairs) {
            const int next = pair + G;
            fetch_tables(next, tn);
            load_pair<BITS>(qn, qweight + (size_t)(2 * next) * W, plane_stride, lane_off);
            float tot[2][M];
            compute(q, tables[0], tot);
            publish(tot);
            lds_only_barrier();  // every wave is done with the tables; segment sums visible
            stage_tables(tn, tables[0]);
            combine(pair);
            lds_only_barrier();  // next tables visible; segment sums consumed
            q = qn;
            pair = next;
        }
        float tot[2][M];
        compute(q, tables[0], tot);
        publish(tot);
        lds_only_barrier();
        combine(pair);
    }
}

}  // namespace ap

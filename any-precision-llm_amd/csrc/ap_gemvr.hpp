// Persistent bitplane GEMV for gfx950, 1 <= M <= 4, rows of a multiple of 64 elements:
//     out[m,n] = sum_k x[m,k] * lut[n, index_b(n,k)]      (fp32 accumulate, fp16 out)
//
// Same contract as the reference's matmul_kbit_32 (any_precision/modules/kernels/matmul.cuh:16-167).
// A launch of one wave per lane-word costs a wave launch per 2048 weights, and the machine starts about
// one wave per 2-3 cycles and XCD: on the MLP shapes of a 7B model that alone is 2.5 us.  Here the grid
// is a few waves per SIMD and every wave LOOPS over rows:
//   * a workgroup is the S waves that cover one row (wave s owns words 128 s .. 128 s + 127, two words
//     per lane, one 8-byte load per plane) and walks the rows g, g + G, ...; its 32 activation registers
//     are loaded once;
//   * kDepth rows are in flight ahead of the one being computed (planes and table), so a wave always has
//     loads outstanding and the stream does not stop while it computes; one row per step keeps the steps
//     short, which is what bounds the un-overlapped start (first loads) and end (last compute);
//   * with S = 1 a workgroup is a single wave: no barrier anywhere, the next table overwrites the current
//     one in place (the LDS executes the operations of one wave in order).  With S > 1 two LDS-only
//     barriers per row order the table and the exchange of the segment sums, added in wave order.
#pragma once
#include "ap_gemvr_launch.hpp"
#include "ap_lookup.hpp"

namespace ap {

constexpr int kGemvrSegWords = 128;  // words of a row one wave covers
constexpr int kGemvrDepth = 2;       // rows in flight ahead of the current one

template <int BITS>
struct RowInFlight {
    u32x2 q[BITS];
    TableWords<BITS> t;
};

// Grid: G <= N workgroups of (64, S) threads, S = ceil(K / 4096) <= THREADS / 64.  K a multiple of 64.
template <int BITS, int M, int THREADS>
__global__ __launch_bounds__(THREADS) void gemvr_kbit_kernel(const half_t *__restrict__ x,
                                                            const uint32_t *__restrict__ qweight,
                                                            const half_t *__restrict__ lut, half_t *__restrict__ out,
                                                            int N, int K) {
    constexpr int NC = 1 << BITS;
    constexpr bool kMulti = THREADS > kWave;
    constexpr int MAXS = THREADS / kWave;
    __shared__ __attribute__((aligned(16))) uint8_t tables[1][LookupTable<BITS>::kBytes];
    __shared__ float partial[MAXS][M];

    const int lane = threadIdx.x;
    const int s = kMulti ? __builtin_amdgcn_readfirstlane(threadIdx.y) : 0;
    const int S = kMulti ? (int)blockDim.y : 1;
    const int W = K >> 5;
    const size_t plane_stride = (size_t)N * W;
    const int G = gridDim.x;

    const uint32_t seg_word = (uint32_t)s * kGemvrSegWords + 2u * (uint32_t)lane;
    const bool valid = seg_word < (uint32_t)W;          // lanes past the row end idle (sums dropped)
    const uint32_t w0 = valid ? seg_word : 0u;
    const PairLane<BITS> pl = pair_lane<BITS>(lane);

    // Rows past the end are replaced by row 0: a few re-reads that hit the cache instead of a second code
    // path (which would merge the load counters of both and make every step wait for everything).
    auto fetch = [&](RowInFlight<BITS> &f, int row) {
        const int r = row < N ? row : 0;
        if (s == 0) f.t = lookup_table_fetch<BITS>(lut + (size_t)r * NC, lane, pl);
        const uint32_t *base = qweight + (size_t)r * W + w0;
#pragma unroll
        for (int p = 0; p < BITS; p++)  // streamed once: non-temporal, so x and the tables keep their cache lines
            f.q[p] = __builtin_nontemporal_load(reinterpret_cast<const u32x2 *>(base + p * plane_stride));
    };

    int row = blockIdx.x;  // the grid never exceeds the number of rows
    RowInFlight<BITS> f[kGemvrDepth + 1];
    // Issue order: first row, activations, the rows behind it.  The first step then waits for exactly as
    // many loads as every later step (the kDepth rows behind the current one stay in flight); with the
    // activations issued last it would have to wait for everything, and -- the load counters of the loop
    // entry and of the loop back-edge being merged -- so would every third step after it.
    fetch(f[0], row);
    uint32_t X[M][2][4][4];
    load_activations_plain<M, 2>(x, K, (int)w0, X);
    __builtin_amdgcn_sched_barrier(0);  // the scheduler would otherwise move the activation loads to the end
#pragma unroll
    for (int d = 1; d <= kGemvrDepth; d++) fetch(f[d], row + d * G);

    // One row from in-flight slot K; the slot is refilled with the row kDepth + 1 steps ahead as soon as its
    // words are used up.  The loop below is unrolled over the slots, so no register ever has to be copied
    // from a load that was issued a moment ago (which would mean waiting for it).  Returns false after the
    // last row.
    int done[M];  // lane i: fp32 bits of the result of this wave's i-th row (single-wave workgroups)
#pragma unroll
    for (int m = 0; m < M; m++) done[m] = 0;
    int it = 0;
    const int first_row = row;
    auto step = [&](auto k_c) -> bool {
        constexpr int k = decltype(k_c)::value;
        if (s == 0) lookup_table_stage<BITS>(f[k].t, tables[0], lane);  // in-order LDS: after the previous row's lookups
        if constexpr (kMulti) lds_only_barrier(); else __builtin_amdgcn_wave_barrier();
        uint32_t words[2][BITS];
#pragma unroll
        for (int p = 0; p < BITS; p++) {
            words[0][p] = f[k].q[p][0];
            words[1][p] = f[k].q[p][1];
        }
        float acc[1][M][2];
#pragma unroll
        for (int m = 0; m < M; m++) acc[0][m][0] = acc[0][m][1] = 0.f;
        lookup_dot<BITS, M, 2, 1, 2>(words, tables, X, acc, [](auto) { return std::integral_constant<int, 0>{}; },
                                     [](auto n) { return n; });
        // refill the slot once its words are used up: the loads land in the registers just freed, so
        // nothing has to be copied (a copy would wait for the load); kDepth rows stay in flight meanwhile
        __builtin_amdgcn_sched_barrier(0);
        fetch(f[k], row + (kGemvrDepth + 1) * G);
        float tot[M];
#pragma unroll
        for (int m = 0; m < M; m++) {
            float v = acc[0][m][0] + acc[0][m][1];
            asm volatile("" : "+v"(v));  // keeps the lookup stream out of an "if (valid)" region
            tot[m] = wave_sum(valid ? v : 0.f);
        }
        if constexpr (!kMulti) {
            // Results are parked in lane `it` of a register and stored after the loop: a store inside it
            // shares the load counter, and with loads and stores both pending the compiler has to wait
            // for ALL of them at the next use of a loaded register, which empties the prefetch queue.
#pragma unroll
            for (int m = 0; m < M; m++) {
                const int total = __builtin_amdgcn_readlane(__builtin_bit_cast(int, tot[m]), kSumLane);
                done[m] = lane == it ? total : done[m];
            }
            it++;
        } else {
            if (lane == kSumLane) {
#pragma unroll
                for (int m = 0; m < M; m++) partial[s][m] = tot[m];
            }
            lds_only_barrier();  // every wave is done with the table; segment sums visible
            if (s == 0 && lane < M) {
                float v = 0.f;
                for (int ss = 0; ss < S; ss++) v += partial[ss][lane];
                out[(size_t)lane * N + row] = (half_t)v;
            }
            // the next step's barrier (after the table is staged) also separates these reads of
            // `partial` from the next writes to it
        }
        row += G;
        return row < N;
    };
    static_assert(kGemvrDepth == 2, "the loop is unrolled over kGemvrDepth + 1 slots");
    while (true) {
        if (!step(std::integral_constant<int, 0>{})) break;
        if (!step(std::integral_constant<int, 1>{})) break;
        if (!step(std::integral_constant<int, 2>{})) break;
    }
    if constexpr (!kMulti) {
        if (lane < it) {  // at most 64 rows per wave (the launch sizes the grid accordingly)
#pragma unroll
            for (int m = 0; m < M; m++)
                out[(size_t)m * N + first_row + (size_t)lane * G] = (half_t)__builtin_bit_cast(float, done[m]);
        }
    }
}

}  // namespace ap

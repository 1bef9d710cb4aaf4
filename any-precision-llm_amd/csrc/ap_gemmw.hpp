// Fused bitplane dequant -> MFMA skinny GEMM that WALKS the weight rows with its activations resident:
//     out[m,n] = sum_k x[m,k] * lut[n, index_b(n,k)]      (fp16 operands, fp32 accumulate), M <= 32
//
// The one-shot kernel (ap_gemm.hpp) gives every block of 16 weight rows its own workgroup of K-split
// waves, and every wave fetches its 16 activation operands per step from L2 again: (N/16) * M * K * 2
// bytes per launch, more than the planes themselves from a few activation rows on, and every wave is one
// long dependent chain (planes -> indices -> 128 lookups -> 16 matrix instructions) with nothing to
// overlap it.  Here a workgroup is the same K-split of waves but lives for the whole launch: a wave loads
// the activation operands of ITS K-slice once (64 registers per 512 elements of K and block of 16
// activation rows) and then walks blocks of 16 weight rows g, g + G, g + 2G, ...; the planes and tables
// of the next block are requested before the current one is looked up, so the memory stream and the
// lookups overlap inside every wave, and the activations are read from L2 once per workgroup.
// The operator is the same as the reference's matmul_kbit / dequant_kbit + matmul
// (any_precision/modules/AnyPrecisionLinear.py:60-64).
//
// Lane mapping, plane loads and the in-wave transposes are those of ap_gemm.hpp: lane l owns weight
// row l % 16 and k-group l / 16; a step is 16 words (512 elements) of every row.  SPW = steps per
// wave (1 or 2), MB = blocks of 16 activation rows; MB * SPW <= 2 bounds the resident operands to 128
// registers.  Requires K % 128 == 0 and at most 8 * SPW steps.
#pragma once
#include <type_traits>

#include "ap_bitplane.hpp"
#include "ap_device.hpp"
#include "ap_gemm.hpp"
#include "ap_gemmw_launch.hpp"
#include "ap_lookup.hpp"

namespace ap {

// Grid: G <= ceil(N / 16) workgroups of (64, KS) threads, KS = ceil(steps / SPW) >= 4.
template <int BITS, int MB, int SPW>
__global__ __launch_bounds__(kGemmMaxSplit *kWave) void gemmw_kbit_kernel(
    const half_t *__restrict__ x, const uint32_t *__restrict__ qweight, const half_t *__restrict__ lut,
    half_t *__restrict__ out, int M, int N, int K) {
    constexpr int NC = 1 << BITS;
    constexpr bool PAIR = LookupTable<BITS>::kPair;  // 3 and 4 bits: tables of adjacent element pairs (ap_lookup.hpp)
    constexpr int TB = LookupTable<BITS>::kBytes;    // bytes of one row's table in LDS
    constexpr int TQ = kGemmRows * NC / 8;  // 16-byte quads of the tables of one block of rows
    constexpr int TPT = 2;                  // of which a thread carries at most two (KS >= 4)
    constexpr int RPW = 4;                  // pair tables: rows a wave builds per block (KS >= 4)
    static_assert(MB * SPW <= 2 && TQ <= TPT * 4 * kWave, "");
    __shared__ __attribute__((aligned(16))) uint8_t tables[2][kGemmRows][TB];
    __shared__ float part[2][kGemmMaxSplit][MB * 4 * kWave];

    const int lane = threadIdx.x;
    const int ks = __builtin_amdgcn_readfirstlane(threadIdx.y), KS = blockDim.y;
    const int tid = ks * kWave + lane, nthr = KS * kWave;
    const int col = lane & 15, grp = lane >> 4;
    const int W = K >> 5;
    const size_t plane_stride = (size_t)N * W;
    const int steps = (W + 15) >> 4;
    const int nblocks = (N + kGemmRows - 1) / kGemmRows;
    const int full_chunks = W >> 5;
    const uint32_t tail_stride = (uint32_t)(W & 31) * 16u;

    typedef __attribute__((address_space(3))) half_t lds_half_t;
    typedef __attribute__((address_space(3))) uint32_t lds_u32_t;
    uint32_t tab_base[2];
#pragma unroll
    for (int b = 0; b < 2; b++)
        tab_base[b] = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) uint8_t *)&tables[b][0][0]) + (uint32_t)col * TB;
    const PairLane<BITS> pl = pair_lane<BITS>(lane);

    // ---- the activation operands of this wave's steps, once.  Word wi of step s is w = 16 step + 4 wi + grp;
    // its byte group j multiplies x[m][kb + j * jstride .. +7].  Words past the row end get zeros (their
    // weights are zeroed too).
    half8_t a[SPW][16][MB];
    uint32_t livemask = 0u;  // bit 4 s + wi
#pragma unroll
    for (int s = 0; s < SPW; s++) {
        const int step = ks * SPW + s;
#pragma unroll
        for (int wi = 0; wi < 4; wi++) {
            const int w = 16 * step + 4 * wi + grp;
            const bool live = step < steps && w < W;
            livemask |= (live ? 1u : 0u) << (4 * s + wi);
            const int wc = live ? w : 0;
            const int chunk = wc >> 5;
            const uint32_t kb = ((uint32_t)chunk << 11) + ((uint32_t)(wc & 31) << 4);
            const uint32_t jstride = chunk == full_chunks ? tail_stride : 512u;
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int mb = 0; mb < MB; mb++) {
                    const uint32_t off = (uint32_t)min(mb * 16 + col, M - 1) * (uint32_t)K * 2u + kb + (uint32_t)j * jstride;
                    const half8_t v = *reinterpret_cast<const half8_t *>(reinterpret_cast<const char *>(x) + (size_t)off);
                    a[s][4 * wi + j][mb] = live ? v : half8_t{0, 0, 0, 0, 0, 0, 0, 0};
                }
        }
    }

    // planes of block `blk` for this wave's steps (16-byte loads; steps past the row are clamped and unused)
    auto fetch = [&](int blk, uint32_t(&q)[SPW][BITS][4]) {
        const uint32_t *wrow = qweight + (size_t)min(blk * kGemmRows + col, N - 1) * W;
#pragma unroll
        for (int s = 0; s < SPW; s++) {
            const int w = min(16 * (ks * SPW + s) + 4 * grp, W - 4);
#pragma unroll
            for (int p = 0; p < BITS; p++) {
                const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(wrow + p * plane_stride + w));
#pragma unroll
                for (int i = 0; i < 4; i++) q[s][p][i] = v[i];
            }
        }
    };
    // tables of block `blk`: contiguous in lut (rows past N re-read the last quad; their columns are never stored)
    // pair tables: wave ks builds those of rows ks, ks + KS, ... of the block
    struct TableRegs {
        u32x4 v[PAIR ? 1 : TPT];
        TableWords<BITS> w[PAIR ? RPW : 1];
    };
    auto table_fetch = [&](int blk) {
        TableRegs r;
        if constexpr (PAIR) {
#pragma unroll
            for (int i = 0; i < RPW; i++) {
                const int row = min(blk * kGemmRows + min(ks + i * KS, kGemmRows - 1), N - 1);
                r.w[i] = lookup_table_fetch<BITS>(lut + (size_t)row * NC, lane, pl);
            }
        } else {
            const u32x4 *src = reinterpret_cast<const u32x4 *>(lut);
            const long long first = (long long)blk * TQ, last = (long long)N * (NC / 8) - 1;
#pragma unroll
            for (int i = 0; i < TPT; i++) {
                const int e = tid + i * nthr;
                r.v[i] = src[min(first + min(e, TQ - 1), last)];
            }
        }
        return r;
    };
    auto table_stage = [&](const TableRegs &r, int slot) {
        if constexpr (PAIR) {
#pragma unroll
            for (int i = 0; i < RPW; i++)
                if (ks + i * KS < kGemmRows) lookup_table_stage<BITS>(r.w[i], &tables[slot][ks + i * KS][0], lane);
        } else {
            u32x4 *dst = reinterpret_cast<u32x4 *>(&tables[slot][0][0]);
#pragma unroll
            for (int i = 0; i < TPT; i++) {
                const int e = tid + i * nthr;
                if (e < TQ) dst[e] = r.v[i];
            }
        }
    };

    // One block of 16 weight rows against the resident operands; the partial tile goes to part[slot][ks].
    constexpr int PRE = BITS <= 7 ? 1 : 0;  // index bytes hold the table byte offset where that fits a byte
    auto compute = [&](uint32_t(&q)[SPW][BITS][4], int slot) {
        float4_t acc[MB];
#pragma unroll
        for (int mb = 0; mb < MB; mb++) acc[mb] = float4_t{0.f, 0.f, 0.f, 0.f};
        const uint32_t tbase = tab_base[slot];
        static_for<SPW>([&](auto s_c) {
            constexpr int s = decltype(s_c)::value;
            if (ks * SPW + s < steps) {
#pragma unroll
                for (int p = 0; p < BITS; p++) transpose_rows4(q[s][p]);
                uint32_t idx[PAIR ? 4 : 8];
                static_for<16>([&](auto t_c) {
                    constexpr int t = decltype(t_c)::value, wi = t / 4, j = t % 4, c = 3 - j;
                    if constexpr (j == 0) {
                        uint32_t qq[BITS];
#pragma unroll
                        for (int p = 0; p < BITS; p++) qq[p] = q[s][p][wi];
                        if constexpr (PAIR) planes_to_adjacent_pairs<BITS>(qq, idx);
                        else planes_to_indices<BITS, PRE>(qq, idx);
                    }
                    const bool live = (livemask >> (4 * s + wi)) & 1u;
                    u32x4 bw;
                    static_for<4>([&](auto e_c) {
                        constexpr int i = decltype(e_c)::value;
                        uint32_t packed;
                        if constexpr (PAIR) {
                            uint32_t a0;
                            if constexpr (BITS == 3) a0 = byte_add<c>(tbase, idx[i]);
                            else a0 = tbase + byte_offset<c, 2>(idx[i]);
                            packed = *reinterpret_cast<const lds_u32_t *>(a0);
                        } else {
                            uint32_t a0, a1;
                            if constexpr (PRE) {
                                a0 = byte_add<c>(tbase, idx[2 * i]);
                                a1 = byte_add<c>(tbase, idx[2 * i + 1]);
                            } else {
                                a0 = tbase + byte_offset<c, 1>(idx[2 * i]);
                                a1 = tbase + byte_offset<c, 1>(idx[2 * i + 1]);
                            }
                            half2_t h;
                            h.x = *reinterpret_cast<const lds_half_t *>(a0);
                            h.y = *reinterpret_cast<const lds_half_t *>(a1);
                            packed = __builtin_bit_cast(uint32_t, h);
                        }
                        bw[i] = live ? packed : 0u;
                    });
                    const half8_t bfrag = __builtin_bit_cast(half8_t, bw);
#pragma unroll
                    for (int mb = 0; mb < MB; mb++)
                        acc[mb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[s][t][mb], bfrag, acc[mb], 0, 0, 0);
                });
            }
        });
        float *mine = &part[slot][ks][0];
#pragma unroll
        for (int mb = 0; mb < MB; mb++)
#pragma unroll
            for (int v = 0; v < 4; v++) mine[(mb * 4 + v) * kWave + lane] = acc[mb][v];
    };
    // Sum of the K-split partial tiles in wave order.  D[i][j]: lane l holds rows i = 4 (l / 16) + v, column l % 16.
    // A wave takes tiles ks and ks + KS (KS >= 4 covers the at most 8 tiles): a fixed number of predicated
    // stores, so the loads already in flight for the next block can be counted past them.
    auto combine = [&](int blk, int slot) {
#pragma unroll
        for (int r = 0; r < 2; r++) {
            const int t = ks + r * KS;
            const bool mine = t < MB * 4;
            const int tc = mine ? t : 0;
            float sum = 0.f;
            for (int kk = 0; kk < KS; kk++) sum += part[slot][kk][tc * kWave + lane];
            const int m = (tc >> 2) * 16 + 4 * grp + (tc & 3), n = blk * kGemmRows + col;
            if (mine && m < M && n < N) out[(size_t)m * N + n] = (half_t)sum;
        }
    };

    // ---- the walk.  Iteration i computes block b_i from tables[i & 1] while the planes and tables of b_{i+1}
    // are in flight; one barrier per block makes the partial tiles of b_i and the tables of b_{i+1} visible.
    // Past the last block the "next" block is the last one again (loads that nobody uses keep the loop one
    // straight path, which is what lets the compiler leave the loads in flight across it).
    const int G = gridDim.x;
    uint32_t q0[SPW][BITS][4], q1[SPW][BITS][4];
    int blk = blockIdx.x;
    fetch(blk, q0);
    table_stage(table_fetch(blk), 0);
    lds_only_barrier();
    for (;;) {
        {   // even iteration: q0, slot 0; prefetch into q1, slot 1
            const int nxt = blk + G < nblocks ? blk + G : blk;
            fetch(nxt, q1);
            const TableRegs tr = table_fetch(nxt);
            compute(q0, 0);
            table_stage(tr, 1);
            lds_only_barrier();
            combine(blk, 0);
            blk += G;
            if (blk >= nblocks) break;
        }
        {   // odd iteration: q1, slot 1; prefetch into q0, slot 0
            const int nxt = blk + G < nblocks ? blk + G : blk;
            fetch(nxt, q0);
            const TableRegs tr = table_fetch(nxt);
            compute(q1, 1);
            table_stage(tr, 0);
            lds_only_barrier();
            combine(blk, 1);
            blk += G;
            if (blk >= nblocks) break;
        }
    }
}

}  // namespace ap

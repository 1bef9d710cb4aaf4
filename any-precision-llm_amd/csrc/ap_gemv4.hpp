// Bitplane skinny GEMM for gfx950 on the 4x4x4 matrix cores, up to 4 MG activation rows
// (used for 3 and 4 rows, and for 5..8 rows on wide linears with rows of about 4096 elements,
// where it beats both other kernels):
//     out[m,n] = sum_k x[m,k] * lut[n, index_b(n,k)]      (fp16 operands, fp32 accumulate)
//
// Same operator as the reference's matmul_kbit_32 with multi_row (any_precision/modules/
// kernels/matmul.cuh:16-167, M > 1 at :25,78-81).  The dot-product kernel (ap_gemv.hpp) pays
// one v_dot2c per weight pair and activation row, so from three rows on it is bound by
// vector ALU issue, not by memory; the 16x16x32 MFMA kernel (ap_gemm.hpp) re-reads the
// activations once per 16 weight rows.  v_mfma_f32_4x4x4_16B_f16 fits in between: it
// multiplies 16 independent 4x4x4 blocks, one block per 4 adjacent lanes.
//
// Mapping: lane l = (block wb = l / 4, row qi = l % 4).  A wave owns four weight rows
// r0 .. r0+3 and, per word group g, the sixteen words 16 (s G + g) .. +15 of each; lane
// (wb, qi) owns word wb of row r0 + qi.  It rebuilds the 32 indices of its word, gathers from
// its row's table in LDS and has, per byte group, eight consecutive-k weights: two B
// operands (k 0..3 and 4..7; B[k][j]: lane (blk, j) supplies column j = its weight row).
// The A operand is x[m][same eight k] with m = l % 4 (A[i][k]: lane (blk, i) supplies row
// i = activation row): the four lanes of a block cover the same k range, so every lane
// loads the activations of "its" word once, for one activation row, and the matrix core
// does the 4 x 4 cross product.  D[i][j] lands in lane (blk, j) as four registers i = 0..3:
// each lane accumulates the dot products of its own weight row with four activation rows.
// Cost per weight does not depend on M.
//
// A workgroup is the S waves (S = ceil(W / (16 G))) of RQ consecutive row quads; a wave keeps
// its activations in registers and walks the RQ quads with them, so the activations are
// read from L2 once per 4 RQ weight rows -- at M rows that traffic is M / (2 RQ) bytes per
// weight against w_bits / 8 from HBM, and it, not the arithmetic, is what a small RQ pays
// for.  Partial sums meet in LDS and are added in a fixed order.
#pragma once
#include <type_traits>

#include "ap_bitplane.hpp"
#include "ap_device.hpp"
#include "ap_gemv4_launch.hpp"
#include "ap_lookup.hpp"

namespace ap {

typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

// MG = groups of four activation rows (M <= 4 MG), G = word groups per wave, RQ = row quads
// per workgroup.  Grid: ceil(N / (4 RQ)) workgroups of (64, S) threads, S * 64 <= THREADS (S is also an argument: it
// arrives with the others instead of through a load of its own from the dispatch packet).
template <int BITS, int MG, int G, int RQ, int THREADS>
__global__ __launch_bounds__(THREADS) void gemv4_kbit_kernel(
    const half_t *__restrict__ x, const uint32_t *__restrict__ qweight, const half_t *__restrict__ lut,
    half_t *__restrict__ out, int M, int N, int K, int S) {
    constexpr int NC = 1 << BITS;
    constexpr int MAXS = THREADS / kWave;
    constexpr int MR = 4 * MG;  // activation rows computed (rows past M repeat row M-1 and are not stored)
    constexpr int ROWS = 4 * RQ;
    // 3 and 4 bits: tables of the weights of two ADJACENT elements (ap_lookup.hpp) -- one 32-bit gather per half of a
    // B operand, no packing of two 16-bit gathers, and the entry numbers come out of a shorter transpose
    // (planes_to_adjacent_pairs).  The activations stay as they sit in memory.
    constexpr bool PAIR = LookupTable<BITS>::kPair;
    constexpr int TB = LookupTable<BITS>::kBytes;
    __shared__ __attribute__((aligned(16))) uint8_t tables[ROWS][TB];
    __shared__ float partial[MAXS][ROWS][MR];  // [wave][weight row][activation row]

    // every argument in scalar registers by one clause of scalar loads and one wait (the compiler alone loads an
    // argument where it is first used: a dependent round trip to the scalar cache each)
    asm volatile("" : "+s"(x), "+s"(qweight), "+s"(lut), "+s"(out), "+s"(M), "+s"(N), "+s"(K), "+s"(S));
    const int lane = threadIdx.x;
    const int s = __builtin_amdgcn_readfirstlane(threadIdx.y);
    const int qi = lane & 3, wb = lane >> 2;
    const int W = K >> 5;
    const size_t plane_bytes = (size_t)N * W * sizeof(uint32_t);  // below 2^32 (the host checks)
    const int row0 = blockIdx.x * ROWS;
    // loads are a scalar base plus a 32-bit byte offset per lane (no 64-bit vector arithmetic per load)
    const global_ptr<const char> qbytes = scalar_ptr(reinterpret_cast<const char *>(qweight));
    const global_ptr<const half_t> xg = scalar_ptr(x);

    // Load order as in the dot-product kernel: tables, planes (non-temporal: streamed once),
    // activations.
    // wave s stages the tables of rows s, s + S, ...: with the usual eight waves for eight rows one each, found
    // without a chain of per-row branches (whose address arithmetic would run for every row, ahead of the first load)
    const PairLane<BITS> pl = pair_lane<BITS>(lane);
    const global_ptr<const half_t> lut_g = scalar_ptr(lut);
    TableWords<BITS> t[ROWS];
#pragma unroll
    for (int i = 0; i < ROWS; i++) {
        const int r = s + i * S;
        if (r >= ROWS) break;
        t[i] = lookup_table_fetch<BITS>(scalar_ptr(lut_g + (size_t)min(row0 + r, N - 1) * NC), lane, pl);
    }

    uint32_t q[RQ][G][BITS];
    bool live[G];
    int wl[G];
#pragma unroll
    for (int g = 0; g < G; g++) {
        const int w = (s * G + g) * 16 + wb;
        live[g] = w < W;
        wl[g] = live[g] ? w : 0;
    }
    // The planes are loaded with lane = (row l / 16, word l % 16), 64 contiguous bytes per row and
    // 16 lanes, and then moved to the block layout (lane 4 wb + qi takes what lane 16 qi + wb
    // loaded) with one cross-lane permute per plane word.
    const int lrow = lane >> 4, lword = lane & 15;
    const int take = (16 * qi + wb) * 4;  // byte address of the source lane for ds_bpermute
#pragma unroll
    for (int rq = 0; rq < RQ; rq++) {
        // rows past N repeat row N-1 and are not stored
        const uint32_t row_words = (uint32_t)min(row0 + 4 * rq + lrow, N - 1) * (uint32_t)W;
#pragma unroll
        for (int g = 0; g < G; g++) {
            const uint32_t byte = (row_words + (uint32_t)min((s * G + g) * 16 + lword, W - 1)) * (uint32_t)sizeof(uint32_t);
#pragma unroll
            for (int p = 0; p < BITS; p++) q[rq][g][p] = load_at_nt<uint32_t>(scalar_ptr(qbytes + p * plane_bytes), byte);
        }
    }
    // X[mg][g][j]: the eight activations of byte group j of this lane's word, row 4 mg + qi
    u32x4 X[MG][G][4];
#pragma unroll
    for (int mg = 0; mg < MG; mg++) {
        const uint32_t xrow = (uint32_t)min(mg * 4 + qi, M - 1) * (uint32_t)K;  // M * K * 2 < 2^32 (M <= 8)
#pragma unroll
        for (int g = 0; g < G; g++)
#pragma unroll
            for (int j = 0; j < 4; j++)
                X[mg][g][j] = load_at<u32x4>(xg, (xrow + (uint32_t)group_base(wl[g], j, K)) * (uint32_t)sizeof(half_t));
    }
    // words past the row end (last wave of a row only): all four lanes of their block are past it,
    // so zero activations silence the whole block
    if ((s * G + G) * 16 > W) {
#pragma unroll
        for (int mg = 0; mg < MG; mg++)
#pragma unroll
            for (int g = 0; g < G; g++)
#pragma unroll
                for (int j = 0; j < 4; j++)
                    if (!live[g]) X[mg][g][j] = u32x4{0u, 0u, 0u, 0u};
    }

#pragma unroll
    for (int i = 0; i < ROWS; i++) {
        const int r = s + i * S;
        if (r >= ROWS) break;
        lookup_table_arrive<BITS>(t[i]);
        lookup_table_stage<BITS>(t[i], tables[r], lane);
    }
    if (S > 1) __syncthreads(); else __builtin_amdgcn_wave_barrier();

    // LDS byte address of this lane's table (LDS pointers are 32-bit offsets)
    typedef __attribute__((address_space(3))) uint8_t lds_byte_t;
    const uint32_t tab_base0 = (uint32_t)(uintptr_t)((lds_byte_t *)&tables[0][0]) + (uint32_t)qi * TB;

    // CHECK: this wave's words may reach past the row end (the last wave of a row only); every other wave runs the copy
    // without the per-lookup selects (a scalar branch).
    auto compute = [&](auto check_c) {
    constexpr bool CHECK = decltype(check_c)::value;
    static_for<RQ>([&](auto rq_c) {
    constexpr int rq = decltype(rq_c)::value;
    const uint32_t tab_base = tab_base0 + rq * 4 * TB;
    f32x4_t acc[MG];
#pragma unroll
    for (int mg = 0; mg < MG; mg++) acc[mg] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    static_for<G>([&](auto g_c) {
        constexpr int g = decltype(g_c)::value;
        uint32_t qq[BITS];
#pragma unroll
        for (int p = 0; p < BITS; p++) qq[p] = (uint32_t)__builtin_amdgcn_ds_bpermute(take, (int)q[rq][g][p]);
        // index bytes hold the byte offset into the table (index * 2) where that fits a byte
        constexpr int PRE = BITS <= 7 ? 1 : 0;
        uint32_t idx[PAIR ? 4 : 8];
        if constexpr (PAIR) planes_to_adjacent_pairs<BITS>(qq, idx);
        else planes_to_indices<BITS, PRE>(qq, idx);
        static_for<4>([&](auto j_c) {
            constexpr int j = decltype(j_c)::value, c = 3 - j;
            uint32_t bw[4];  // the eight weights of byte group j, two per register
            static_for<4>([&](auto e_c) {
                constexpr int i = decltype(e_c)::value;
                uint32_t packed;
                if constexpr (PAIR) {
                    // byte c of idx[i]: the entry of elements (2i, 2i+1) of byte group j -- at 3 bits already its byte offset
                    uint32_t a0;
                    if constexpr (BITS == 3) a0 = byte_add<c>(tab_base, idx[i]);
                    else a0 = tab_base + byte_offset<c, 2>(idx[i]);
                    packed = *reinterpret_cast<const __attribute__((address_space(3))) uint32_t *>(a0);
                } else {
                    uint32_t a0, a1;
                    if constexpr (PRE) {
                        a0 = byte_add<c>(tab_base, idx[2 * i]);
                        a1 = byte_add<c>(tab_base, idx[2 * i + 1]);
                    } else {
                        a0 = tab_base + byte_offset<c, 1>(idx[2 * i]);
                        a1 = tab_base + byte_offset<c, 1>(idx[2 * i + 1]);
                    }
                    const uint32_t lo = *reinterpret_cast<const __attribute__((address_space(3))) uint16_t *>(a0);
                    const uint32_t hi = *reinterpret_cast<const __attribute__((address_space(3))) uint16_t *>(a1);
                    packed = lo | (hi << 16);
                }
                // words past the row end: zero weights as well as zero activations, so that a non-finite
                // table entry or activation there cannot turn 0 * inf into NaN
                bw[i] = !CHECK || live[g] ? packed : 0u;
            });
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const half4_t bfrag = __builtin_bit_cast(half4_t, u32x2{bw[2 * h], bw[2 * h + 1]});
#pragma unroll
                for (int mg = 0; mg < MG; mg++) {
                    const half4_t afrag = __builtin_bit_cast(half4_t, u32x2{X[mg][g][j][2 * h], X[mg][g][j][2 * h + 1]});
                    acc[mg] = __builtin_amdgcn_mfma_f32_4x4x4f16(afrag, bfrag, acc[mg], 0, 0, 0);
                }
            }
        });
    });

    // Sum over the 16 blocks, i.e. over the lanes with the same l % 4.  Two shifted adds within each
    // 16-lane row leave the row's sums in its lanes 12..15; the four rows are then folded with
    // half / quarter swaps BETWEEN the four accumulators, so that one add serves two of them:
    // afterwards row r of `u` holds the total of accumulator kOrder[r].
#pragma unroll
    for (int mg = 0; mg < MG; mg++) {
        uint32_t v[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            float f = acc[mg][i];
            f = dpp_add<0x114>(f);  // row_shr:4
            f = dpp_add<0x118>(f);  // row_shr:8
            v[i] = __builtin_bit_cast(uint32_t, f);
        }
        auto fold32 = [](uint32_t a, uint32_t b) {  // rows 0,1: a(0+2, 1+3); rows 2,3: b(0+2, 1+3)
            const auto h = __builtin_amdgcn_permlane32_swap(a, b, false, false);
            return __builtin_bit_cast(float, (uint32_t)h[0]) + __builtin_bit_cast(float, (uint32_t)h[1]);
        };
        const float t01 = fold32(v[0], v[1]), t23 = fold32(v[2], v[3]);
        const auto qd = __builtin_amdgcn_permlane16_swap(__builtin_bit_cast(uint32_t, t01), __builtin_bit_cast(uint32_t, t23),
                                                         false, false);
        const float u = __builtin_bit_cast(float, (uint32_t)qd[0]) + __builtin_bit_cast(float, (uint32_t)qd[1]);
        // rows 0..3 of u: totals of accumulators 0, 2, 1, 3
        const int r16 = lane >> 4;
        const int which = ((r16 & 1) << 1) | (r16 >> 1);
        if ((lane & 15) >= 12) partial[s][4 * rq + qi][mg * 4 + which] = u;
    }
    });
    };
    // (only the variant of one word group and four activation rows has the registers for two copies: the others
    // would cross a step of the occupancy table)
    if (G > 1 || MG > 1 || (s * G + G) * 16 > W) compute(std::true_type{});
    else compute(std::false_type{});
    __syncthreads();
    const global_ptr<half_t> out_g = (global_ptr<half_t>)reinterpret_cast<uint64_t>(out);  // a global store, not a flat one
    for (int o = s * kWave + lane; o < ROWS * MR; o += S * kWave) {
        const int m = o % MR, r = o / MR;
        float v = 0.f;
        for (int ss = 0; ss < S; ss++) v += partial[ss][r][m];
        if (m < M && row0 + r < N) out_g[(size_t)m * N + row0 + r] = (half_t)v;
    }
}

}  // namespace ap

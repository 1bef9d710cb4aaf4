// Bitplane GEMV / skinny GEMM for gfx950, 1 <= M <= 8:
//     out[m,n] = sum_k x[m,k] * lut[n, index_b(n,k)]      (fp32 accumulate, fp16 out)
//
// Replaces the reference's matmul_kbit_32<maxm,bits,use_ksplit>
// (any_precision/modules/kernels/matmul.cuh:16-167); the reference sums in
// fp16, this kernel in fp32.
//
// Per weight the path costs a table lookup, so besides HBM it loads the VALU and the LDS
// gather pipe; the design minimises instructions per weight and keeps every wave short:
//   * A workgroup is the S waves of R consecutive rows; wave s owns K-segment s (64*WPL
//     consecutive words = 2048*WPL elements).  The row's table sits at a compile-time LDS
//     address and a gather address is a single SDWA byte-extract-and-shift.
//   * The activations a lane needs are the same for every row: they are loaded into
//     registers once, as they sit in memory.
//   * Per row a lane streams WPL words per plane (one load per plane, a wave covers
//     256*WPL contiguous bytes), rebuilds its indices with a butterfly transpose in
//     registers, gathers from LDS and feeds v_dot2c_f32_f16.
//   * 3 and 4 bits use a pair table (reference idea: matmul.cuh:24,41-49,
//     dequant.cuh:13-30,56-67) of two ADJACENT elements (ap_lookup.hpp): 4^b entries of
//     two fp16, one 32-bit gather per two weights and no packing.  5..8 bits gather single
//     fp16 entries and pack two of them per dot2.
//   * Lane partials are summed with DPP; when S > 1 the segment partials of a row meet in
//     LDS and are added in a fixed order: results are deterministic.
#pragma once
#include <type_traits>

#include "ap_bitplane.hpp"
#include "ap_device.hpp"
#include "ap_gemv_launch.hpp"
#include "ap_lookup.hpp"

namespace ap {


template <int WPL>
struct WordVec;
template <>
struct WordVec<1> { typedef uint32_t type; };
template <>
struct WordVec<2> { typedef u32x2 type; };

template <int WPL>
__device__ __forceinline__ uint32_t word_of(const typename WordVec<WPL>::type &v, int i) {
    if constexpr (WPL == 1) return v; else return v[i];
}

// One row x one lane: rebuild the indices of this lane's WPL words, gather from
// `table` (an LDS array at a compile-time address) and accumulate the M dot products.
template <int BITS, int M, int WPL>
__device__ __forceinline__ void row_dot(const typename WordVec<WPL>::type (&q)[BITS],
                                        const uint8_t (&table)[LookupTable<BITS>::kBytes],
                                        const uint32_t (&X)[M][WPL][4][4], float (&acc)[M][2]) {
#pragma unroll
    for (int wi = 0; wi < WPL; wi++) {
        uint32_t qq[BITS];
#pragma unroll
        for (int p = 0; p < BITS; p++) qq[p] = word_of<WPL>(q[p], wi);
        if constexpr (LookupTable<BITS>::kPair) {
            uint32_t apair[4];
            // byte = entry number (4 bits) or the entry's byte offset (3 bits); a table entry is 4 bytes
            planes_to_adjacent_pairs<BITS>(qq, apair);
            auto gather_pair = [&](auto i_c, auto c_c) {
                constexpr int i = decltype(i_c)::value, c = decltype(c_c)::value;
                const uint32_t off = byte_offset<c, BITS == 4 ? 2 : 0>(apair[i]);
                const uint32_t w2 = *reinterpret_cast<const uint32_t *>(&table[off]);
#pragma unroll
                for (int m = 0; m < M; m++) acc[m][c & 1] = dot2(w2, X[m][wi][3 - c][i], acc[m][c & 1]);
            };
            static_for<4>([&](auto i_c) { static_for<4>([&](auto c_c) { gather_pair(i_c, c_c); }); });
        } else {
            uint32_t idx[8];
            planes_to_indices<BITS>(qq, idx);
            auto gather_two = [&](auto i_c, auto c_c) {
                constexpr int i = decltype(i_c)::value, c = decltype(c_c)::value;
                const uint32_t o0 = byte_offset<c, 1>(idx[2 * i]);
                const uint32_t o1 = byte_offset<c, 1>(idx[2 * i + 1]);
                const uint32_t lo = *reinterpret_cast<const uint16_t *>(&table[o0]);
                const uint32_t hi = *reinterpret_cast<const uint16_t *>(&table[o1]);
                const uint32_t w2 = lo | (hi << 16);
#pragma unroll
                for (int m = 0; m < M; m++) acc[m][c & 1] = dot2(w2, X[m][wi][3 - c][i], acc[m][c & 1]);
            };
            static_for<4>([&](auto i_c) { static_for<4>([&](auto c_c) { gather_two(i_c, c_c); }); });
        }
    }
}

// The GEMV kernel.  A workgroup is the S waves of R consecutive rows (R = 1, 2 or 4,
// compile time).  Every wave issues all the global loads it will ever need -- the tables,
// the planes of its R rows, its activations -- before it computes anything, so the
// memory pipe is full from the first cycle and there is no loop-carried prefetch.  Every
// table sits at a compile-time LDS address.
// Grid: ceil(N / R) workgroups per member, of (64, S) threads (S is also an argument: it arrives with the
// others instead of through a load of its own from the dispatch packet); S*64 <= THREADS.  THREADS (256, 512 or
// 1024) only bounds the workgroup size, so that small workgroups may use more registers
// per lane (M x WPL x 16 of them hold the activations).
//
// One launch serves up to kGemvMaxGroup linears that share x, K and the bit-width (the
// q/k/v or gate/up projections of a decoder layer): `mem` lists them and the workgroup
// range of each; a plain call is a set of one.
//
// PAIR (R = 2 only): the two rows of a workgroup are row n of member 0 and row n of member 1 (two linears of
// equal shape), and what is stored is silu(member 0) * member 1 -- the gate and up projections of a SwiGLU
// MLP with their activation function, one output per row pair, nothing written in between.
// Waves per SIMD the register allocator is asked to keep room for (1 = no request).  At 8 bits with two to
// four activation rows the allocator, left alone, settles two or three registers above a step of the
// occupancy table (83 where 80 fit six waves, 99 where 96 fit five) and a workgroup fewer fits the CU; the
// request is what the registers a lane holds by design allow -- 16 per activation row for x, one per plane
// and row, about 14 more -- out of 512 per SIMD lane in blocks of 8.  No instance spills with it; at fewer
// bits the pair-table lookups in flight need more than the estimate, and the allocator does well alone.
constexpr int gemv_waves_per_simd(int bits, int m, int wpl, int r) {
    if (bits != 8 || wpl > 1 || m < 2 || m > 4) return 1;
    const int need = 16 * m + r * bits + 14;
    const int waves = 512 / ((need + 7) / 8 * 8);
    return waves > 8 ? 8 : waves;
}

template <int BITS, int M, int WPL, int R, int THREADS, bool PAIR = false>
__global__ __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(gemv_waves_per_simd(BITS, M, WPL, R))))
void gemv_kbit_kernel(const half_t *__restrict__ x, const GemvMembers mem, int K, int S) {
    static_assert(!PAIR || R == 2, "a pair is two rows");
    constexpr int NC = 1 << BITS;
    constexpr int MAXS = THREADS / kWave;
    typedef typename WordVec<WPL>::type wvec_t;
    __shared__ __attribute__((aligned(16))) uint8_t tables[R][LookupTable<BITS>::kBytes];
    __shared__ float partial[MAXS * R * M];

    // Which member this workgroup belongs to.  Written without branches, so that every kernel argument
    // arrives with the first clause of scalar loads (a branch per member costs a dependent scalar load
    // each) and the selects stay in scalar registers; no indexed access to the arguments.
    const int bid = blockIdx.x;
    // Member 0 (the only one of a plain call; with PAIR also member 1) and the scalars every workgroup
    // needs, named in ONE empty statement that wants them in scalar registers: the compiler then fetches
    // them with its first clause of scalar loads and waits once.  Left alone it loads each argument where
    // it is first used, a dependent round trip to the scalar cache every time.
    const uint32_t *q0 = mem.qweight[0], *q1 = mem.qweight[PAIR ? 1 : 0];
    const uint16_t *lut0 = mem.lut[0], *lut1 = mem.lut[PAIR ? 1 : 0];
    uint16_t *out0 = mem.out[0];
    int n0 = mem.n[0], end0 = mem.wg_end[0], end1 = mem.wg_end[1], end2 = mem.wg_end[2], count = mem.count;
    if constexpr (PAIR)
        asm volatile("" : "+s"(q0), "+s"(q1), "+s"(lut0), "+s"(lut1), "+s"(out0), "+s"(n0), "+s"(K), "+s"(S), "+s"(x));
    else
        asm volatile("" : "+s"(q0), "+s"(lut0), "+s"(out0), "+s"(n0), "+s"(end0), "+s"(end1), "+s"(end2), "+s"(count),
                          "+s"(K), "+s"(S), "+s"(x));
    const uint32_t *__restrict__ qweight = q0;
    const half_t *__restrict__ lut = reinterpret_cast<const half_t *>(lut0);
    half_t *__restrict__ out = reinterpret_cast<half_t *>(out0);
    int N = n0, wg0 = 0;
    if constexpr (!PAIR) {
        if (count > 1) {
            // a launch of several linears (a scalar branch; plain calls skip it): which member the workgroup
            // belongs to, then that member's fields by index -- one more clause of scalar loads, cheaper than
            // selecting each field among four
            int g = bid >= end0 ? 1 : 0;  // wg_end ascends
            g = (count > 2 && bid >= end1) ? 2 : g;
            g = (count > 3 && bid >= end2) ? 3 : g;
            if (g > 0) {
                qweight = mem.qweight[g];
                lut = reinterpret_cast<const half_t *>(mem.lut[g]);
                out = reinterpret_cast<half_t *>(mem.out[g]);
                N = mem.n[g];
                wg0 = g == 1 ? end0 : (g == 2 ? end1 : end2);
            }
        }
    }

    // blockDim.x is the wave size, so threadIdx.y is wave-uniform: say so, to keep row
    // addresses in scalar registers
    const int lane = threadIdx.x;
    const int s = __builtin_amdgcn_readfirstlane(threadIdx.y);
    const int W = K >> 5;
    const uint32_t w0 = (uint32_t)(s * kWave + lane) * WPL;
    const bool valid = w0 < (uint32_t)W;
    const uint32_t wl = valid ? w0 : 0u;  // lanes past the row end read word 0; their sums are dropped
    const int row0 = PAIR ? bid : (bid - wg0) * R;
    // row r of this workgroup: its number, the address of its first plane word and of its table (all
    // wave-uniform: a load is a scalar base plus the lane's 32-bit byte offset)
    const size_t plane_bytes = (size_t)N * W * sizeof(uint32_t);
    const uint32_t lane_bytes = wl * (uint32_t)sizeof(uint32_t);
    const char *plane_row[R];
    global_ptr<const half_t> table_row[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int n = PAIR ? row0 : min(row0 + r, N - 1);
        plane_row[r] = reinterpret_cast<const char *>((PAIR ? (r == 0 ? q0 : q1) : qweight) + (size_t)n * W);
        table_row[r] = scalar_ptr((PAIR ? reinterpret_cast<const half_t *>(r == 0 ? lut0 : lut1) : lut) + (size_t)n * NC);
    }

    // Issue order matters: the tables first (tiny; staging them to LDS then overlaps the
    // plane loads -- issued last, the table was the last thing to arrive and cost 15-20 %),
    // then the planes (HBM: the requests must go out at once), then the activations (L2
    // hits; issued before the planes they cost up to 1 us at 3-5 bits).  Rows past N (last
    // workgroup only) re-read row N-1 and are not stored.
    // wave r % S fetches and stages the table of row r; r < 4, so up to three conditional subtractions
    // instead of a division by a run-time S
    auto stages = [&](int r) {
        int owner = r;
#pragma unroll
        for (int i = 0; i < R - 1; i++) owner = owner >= S ? owner - S : owner;
        return s == owner;
    };
    const PairLane<BITS> pl = pair_lane<BITS>(lane);
    TableWords<BITS> t[R];
#pragma unroll
    for (int r = 0; r < R; r++)
        if (stages(r)) t[r] = lookup_table_fetch<BITS>(table_row[r], lane, pl);
    wvec_t q[R][BITS];
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int p = 0; p < BITS; p++)  // streamed once: non-temporal, so x and the tables keep their cache lines
            q[r][p] = load_at_nt<wvec_t>(scalar_ptr(plane_row[r] + p * plane_bytes), lane_bytes);
    uint32_t X[M][WPL][4][4];
    load_activations_plain<M, WPL>(x, K, (int)wl, X);

#pragma unroll
    for (int r = 0; r < R; r++)
        if (stages(r)) {
            lookup_table_arrive<BITS>(t[r]);
            lookup_table_stage<BITS>(t[r], tables[r], lane);
        }
    if (S > 1) lds_only_barrier(); else __builtin_amdgcn_wave_barrier();

    // stores go through a pointer typed as global memory (the argument pointers left the statement above
    // without an address space, and a store through them would be a flat one)
    const global_ptr<half_t> out_g = (global_ptr<half_t>)reinterpret_cast<uint64_t>(out);
    float tot[R][M];
    static_for<R>([&](auto r_c) {
        constexpr int r = decltype(r_c)::value;
        float acc[M][2];
#pragma unroll
        for (int m = 0; m < M; m++) acc[m][0] = acc[m][1] = 0.f;
        row_dot<BITS, M, WPL>(q[r], tables[r], X, acc);
#pragma unroll
        for (int m = 0; m < M; m++) tot[r][m] = wave_sum(valid ? acc[m][0] + acc[m][1] : 0.f);
    });

    auto swiglu = [](float gate, float up) { return gate / (1.f + __expf(-gate)) * up; };
    if (S == 1) {
        if (lane == kSumLane) {
            if constexpr (PAIR) {
#pragma unroll
                for (int m = 0; m < M; m++) out_g[(size_t)m * N + row0] = (half_t)swiglu(tot[0][m], tot[R - 1][m]);
            } else {
#pragma unroll
                for (int r = 0; r < R; r++)
#pragma unroll
                    for (int m = 0; m < M; m++)
                        if (row0 + r < N) out_g[(size_t)m * N + row0 + r] = (half_t)tot[r][m];
            }
        }
    } else {
        if (lane == kSumLane) {
#pragma unroll
            for (int r = 0; r < R; r++)
#pragma unroll
                for (int m = 0; m < M; m++) partial[(s * R + r) * M + m] = tot[r][m];
        }
        __syncthreads();
        const int tid = s * kWave + lane;
        if constexpr (PAIR) {
            if (tid < M) {
                float g = 0.f, u = 0.f;
                for (int ss = 0; ss < S; ss++) {
                    g += partial[(ss * R) * M + tid];
                    u += partial[(ss * R + R - 1) * M + tid];
                }
                out_g[(size_t)tid * N + row0] = (half_t)swiglu(g, u);
            }
        } else if (tid < R * M) {  // S >= 2 waves hold at least 128 threads >= R * M
            const int m = tid % M, r = tid / M;
            float v = 0.f;
            if (S == 2) {  // rows of up to 4096 elements: both partials in one LDS read instead of a loop of two
                v = partial[r * M + m] + partial[(R + r) * M + m];
            } else {
                for (int ss = 0; ss < S; ss++) v += partial[(ss * R + r) * M + m];
            }
            if (row0 + r < N) out_g[(size_t)m * N + row0 + r] = (half_t)v;
        }
    }
}

}  // namespace ap

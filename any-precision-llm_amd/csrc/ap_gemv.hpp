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
//     registers, already permuted into the order the packed layout scatters elements.
//   * Per row a lane streams WPL words per plane (one load per plane, a wave covers
//     256*WPL contiguous bytes), rebuilds its indices with a butterfly transpose in
//     registers, gathers from LDS and feeds v_dot2c_f32_f16.
//   * 3 and 4 bits use a pair table (reference idea: matmul.cuh:24,41-49,
//     dequant.cuh:13-30,56-67): 4^b entries of two fp16 (w[e], w[e+4]), one 32-bit gather
//     per two weights and no packing.  5..8 bits gather single fp16 entries and pack two of
//     them per dot2.
//   * Lane partials are summed with DPP; when S > 1 the segment partials of a row meet in
//     LDS and are added in a fixed order: results are deterministic.
#pragma once
#include <type_traits>

#include "ap_bitplane.hpp"
#include "ap_device.hpp"
#include "ap_gemv_launch.hpp"

namespace ap {


template <int BITS>
struct GemvTable {
    static constexpr bool kPair = BITS <= 4;
    static constexpr int kBytes = kPair ? (4 << (2 * BITS)) : (2 << BITS);
};

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

// Registers that carry one row's table from global memory to LDS.
template <int BITS>
struct TableRegs {
    uint32_t a;
    u32x2 b;
};

// Issue the global loads of row `lut_row` (2^BITS fp16) for this lane.
template <int BITS>
__device__ __forceinline__ TableRegs<BITS> table_fetch(const half_t *lut_row, int lane) {
    TableRegs<BITS> r;
    r.a = 0u;
    r.b = u32x2{0u, 0u};
    const uint16_t *l16 = reinterpret_cast<const uint16_t *>(lut_row);
    if constexpr (BITS == 3) {          // entry `lane` = (lut[lane >> 3], lut[lane & 7])
        r.a = l16[lane >> 3];
        r.b.x = l16[lane & 7];
    } else if constexpr (BITS == 4) {   // entries 4*lane .. 4*lane+3 = (lut[lane >> 2], lut[4*(lane&3) + i])
        r.a = l16[lane >> 2];
        r.b = reinterpret_cast<const u32x2 *>(lut_row)[lane & 3];
    } else if constexpr (BITS == 8) {   // 512 B: 64 lanes x 8 B
        r.b = reinterpret_cast<const u32x2 *>(lut_row)[lane];
    } else if constexpr (BITS == 7) {   // 256 B: 64 lanes x 4 B
        r.a = reinterpret_cast<const uint32_t *>(lut_row)[lane];
    } else {                            // 64 / 128 B: first lanes x 4 B
        if (lane < (1 << BITS) / 2) r.a = reinterpret_cast<const uint32_t *>(lut_row)[lane];
    }
    return r;
}

// Write the fetched table into LDS in the form the gathers expect.
template <int BITS>
__device__ __forceinline__ void table_stage(const TableRegs<BITS> &r, uint8_t *slot, int lane) {
    if constexpr (BITS == 3) {
        reinterpret_cast<uint32_t *>(slot)[lane] = r.a | (r.b.x << 16);
    } else if constexpr (BITS == 4) {
        u32x4 v;
        v[0] = r.a | (r.b.x << 16);
        v[1] = r.a | (r.b.x & 0xffff0000u);
        v[2] = r.a | (r.b.y << 16);
        v[3] = r.a | (r.b.y & 0xffff0000u);
        reinterpret_cast<u32x4 *>(slot)[lane] = v;
    } else if constexpr (BITS == 8) {
        reinterpret_cast<u32x2 *>(slot)[lane] = r.b;
    } else if constexpr (BITS == 7) {
        reinterpret_cast<uint32_t *>(slot)[lane] = r.a;
    } else {
        if (lane < (1 << BITS) / 2) reinterpret_cast<uint32_t *>(slot)[lane] = r.a;
    }
}

// Workgroup barrier that orders LDS traffic only: outstanding global loads
// (the prefetch of the next row) stay in flight across it.
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// Activations of one lane's words, loaded once per wave.  X[m][wi][j][i] multiplies
// the weight pair gathered for byte group j of word wi: elements (2i, 2i+1) of the
// group, or (i, i+4) in pair-table mode.
template <int BITS, int M, int WPL>
__device__ __forceinline__ void load_activations(const half_t *__restrict__ x, int K, int wl,
                                                 uint32_t (&X)[M][WPL][4][4]) {
#pragma unroll
    for (int m = 0; m < M; m++)
#pragma unroll
        for (int wi = 0; wi < WPL; wi++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const u32x4 v = *reinterpret_cast<const u32x4 *>(x + (size_t)m * K + group_base(wl + wi, j, K));
                if constexpr (GemvTable<BITS>::kPair) {
                    X[m][wi][j][0] = __builtin_amdgcn_perm(v[2], v[0], 0x05040100u);
                    X[m][wi][j][1] = __builtin_amdgcn_perm(v[2], v[0], 0x07060302u);
                    X[m][wi][j][2] = __builtin_amdgcn_perm(v[3], v[1], 0x05040100u);
                    X[m][wi][j][3] = __builtin_amdgcn_perm(v[3], v[1], 0x07060302u);
                } else {
#pragma unroll
                    for (int i = 0; i < 4; i++) X[m][wi][j][i] = v[i];
                }
            }
}

// One row x one lane: rebuild the indices of this lane's WPL words, gather from
// `table` (an LDS array at a compile-time address) and accumulate the M dot products.
template <int BITS, int M, int WPL>
__device__ __forceinline__ void row_dot(const typename WordVec<WPL>::type (&q)[BITS],
                                        const uint8_t (&table)[GemvTable<BITS>::kBytes],
                                        const uint32_t (&X)[M][WPL][4][4], float (&acc)[M][2]) {
#pragma unroll
    for (int wi = 0; wi < WPL; wi++) {
        uint32_t qq[BITS];
#pragma unroll
        for (int p = 0; p < BITS; p++) qq[p] = word_of<WPL>(q[p], wi);
        if constexpr (GemvTable<BITS>::kPair) {
            uint32_t pidx[4];
            // byte = pair index (4 bits) or pair index << 1 (3 bits); a table entry is 4 bytes
            planes_to_pair_indices<BITS, BITS == 3 ? 1 : 0>(qq, pidx);
            auto gather_pair = [&](auto i_c, auto c_c) {
                constexpr int i = decltype(i_c)::value, c = decltype(c_c)::value;
                const uint32_t off = byte_offset<c, BITS == 4 ? 2 : 1>(pidx[i]);
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
// Grid: ceil(N / R) workgroups per member, of (64, S) threads; S*64 <= THREADS.  THREADS (256, 512 or
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
template <int BITS, int M, int WPL, int R, int THREADS, bool PAIR = false>
__global__ __launch_bounds__(THREADS) void gemv_kbit_kernel(const half_t *__restrict__ x, const GemvMembers mem, int K) {
    static_assert(!PAIR || R == 2, "a pair is two rows");
    constexpr int NC = 1 << BITS;
    constexpr int MAXS = THREADS / kWave;
    typedef typename WordVec<WPL>::type wvec_t;
    __shared__ __attribute__((aligned(16))) uint8_t tables[R][GemvTable<BITS>::kBytes];
    __shared__ float partial[MAXS * R * M];

    // which member this workgroup belongs to (scalar selects; no indexed access to the arguments)
    const uint32_t *__restrict__ qweight = mem.qweight[0];
    const half_t *__restrict__ lut = reinterpret_cast<const half_t *>(mem.lut[0]);
    half_t *__restrict__ out = reinterpret_cast<half_t *>(mem.out[0]);
    int N = mem.n[0], wg0 = 0;
#pragma unroll
    for (int g = 1; g < kGemvMaxGroup; g++) {
        if (!PAIR && g < mem.count && (int)blockIdx.x >= mem.wg_end[g - 1]) {
            qweight = mem.qweight[g];
            lut = reinterpret_cast<const half_t *>(mem.lut[g]);
            out = reinterpret_cast<half_t *>(mem.out[g]);
            N = mem.n[g];
            wg0 = mem.wg_end[g - 1];
        }
    }

    // blockDim.x is the wave size, so threadIdx.y is wave-uniform: say so, to keep row
    // addresses in scalar registers
    const int lane = threadIdx.x;
    const int s = __builtin_amdgcn_readfirstlane(threadIdx.y), S = blockDim.y;
    const int W = K >> 5;
    const size_t plane_stride = (size_t)N * W;
    const uint32_t w0 = (uint32_t)(s * kWave + lane) * WPL;
    const bool valid = w0 < (uint32_t)W;
    const uint32_t wl = valid ? w0 : 0u;  // lanes past the row end read word 0; their sums are dropped
    const int row0 = PAIR ? (int)blockIdx.x : ((int)blockIdx.x - wg0) * R;
    // row r of this workgroup: its number, its planes and its tables
    auto row_of = [&](int r) { return PAIR ? row0 : min(row0 + r, N - 1); };
    auto planes_of = [&](int r) { return PAIR ? mem.qweight[r] : qweight; };
    auto tables_of = [&](int r) { return PAIR ? reinterpret_cast<const half_t *>(mem.lut[r]) : lut; };

    // Issue order matters: the tables first (tiny; staging them to LDS then overlaps the
    // plane loads -- issued last, the table was the last thing to arrive and cost 15-20 %),
    // then the planes (HBM: the requests must go out at once), then the activations (L2
    // hits; issued before the planes they cost up to 1 us at 3-5 bits).  Rows past N (last
    // workgroup only) re-read row N-1 and are not stored.
    TableRegs<BITS> t[R];
#pragma unroll
    for (int r = 0; r < R; r++)
        if (s == r % S) t[r] = table_fetch<BITS>(tables_of(r) + (size_t)row_of(r) * NC, lane);
    wvec_t q[R][BITS];
#pragma unroll
    for (int r = 0; r < R; r++) {
        const uint32_t *p0 = planes_of(r) + (size_t)row_of(r) * W;  // uniform per wave
#pragma unroll
        for (int p = 0; p < BITS; p++)  // streamed once: non-temporal, so x and the tables keep their cache lines
            q[r][p] = __builtin_nontemporal_load(reinterpret_cast<const wvec_t *>(p0 + p * plane_stride + wl));
    }
    uint32_t X[M][WPL][4][4];
    load_activations<BITS, M, WPL>(x, K, (int)wl, X);

#pragma unroll
    for (int r = 0; r < R; r++)
        if (s == r % S) table_stage<BITS>(t[r], tables[r], lane);
    if (S > 1) lds_barrier(); else __builtin_amdgcn_wave_barrier();

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
                for (int m = 0; m < M; m++) out[(size_t)m * N + row0] = (half_t)swiglu(tot[0][m], tot[R - 1][m]);
            } else {
#pragma unroll
                for (int r = 0; r < R; r++)
#pragma unroll
                    for (int m = 0; m < M; m++)
                        if (row0 + r < N) out[(size_t)m * N + row0 + r] = (half_t)tot[r][m];
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
                out[(size_t)tid * N + row0] = (half_t)swiglu(g, u);
            }
        } else if (tid < R * M) {  // S >= 2 waves hold at least 128 threads >= R * M
            const int m = tid % M, r = tid / M;
            float v = 0.f;
            for (int ss = 0; ss < S; ss++) v += partial[(ss * R + r) * M + m];
            if (row0 + r < N) out[(size_t)m * N + row0 + r] = (half_t)v;
        }
    }
}

}  // namespace ap

// Table staging and the lookup + dot-product stream shared by the row-pair GEMV kernels
// (ap_gemvp.hpp, ap_gemvf.hpp).
//
// 5..8 bits: the row's table of 2^b fp16 entries is copied to LDS as it is; a lookup is one
// ds_read_u16 and two of them are packed for a v_dot2c_f32_f16.
// 3 and 4 bits: a PAIR table (the reference's idea, any_precision/modules/kernels/matmul.cuh:24,41-49)
// of 4^b dword entries (w[2i], w[2i+1]) -- the weights of two ADJACENT elements, which share a dword of
// the activations, so one ds_read_b32 feeds one v_dot2c_f32_f16 with the activations exactly as they sit
// in memory.  The entry number is the bit-interleaved pair of indices that planes_to_adjacent_pairs
// (ap_bitplane.hpp) produces.
#pragma once
#include "ap_bitplane.hpp"
#include "ap_device.hpp"

namespace ap {

template <int BITS>
struct LookupTable {
    static constexpr bool kPair = BITS <= 4;
    static constexpr int kBytes = kPair ? (4 << (2 * BITS)) : (2 << BITS);
};

// What a lane needs to know to build its share of a pair table; depends on the lane only.
template <int BITS>
struct PairLane {
    uint32_t first, second;  // 3 bits: entry `lane` = (lut[first], lut[second]); 4 bits: dword numbers (below)
};

template <int BITS>
__device__ __forceinline__ PairLane<BITS> pair_lane(int lane) {
    PairLane<BITS> r = {0u, 0u};
    if constexpr (BITS == 3) {
        adjacent_pair_split<3>((uint32_t)lane << 2, r.first, r.second);
    } else if constexpr (BITS == 4) {
        // entries 4*lane .. 4*lane+3 differ in the lowest bit of either index: they combine the halves
        // of dword `first` = (lut[2a], lut[2a+1]) and of dword `second`
        uint32_t a, b;
        adjacent_pair_split<4>((uint32_t)lane << 2, a, b);
        r.first = a >> 1;
        r.second = b >> 1;
    }
    return r;
}

// Registers that carry one row's table from global memory to LDS.
template <int BITS>
struct TableWords {
    uint32_t a, b;
    u32x2 c;
};

// Issue the global loads of row `lut_row` (2^BITS fp16) for this lane: a scalar row address plus the lane's
// 32-bit byte offset.
template <int BITS>
__device__ __forceinline__ TableWords<BITS> lookup_table_fetch(global_ptr<const half_t> lut_row, int lane, const PairLane<BITS> &pl) {
    TableWords<BITS> r;
    r.a = r.b = 0u;
    r.c = u32x2{0u, 0u};
    if constexpr (BITS == 3) {
        r.a = load_at<uint16_t>(lut_row, pl.first * 2u);
        r.b = load_at<uint16_t>(lut_row, pl.second * 2u);
    } else if constexpr (BITS == 4) {
        r.a = load_at<uint32_t>(lut_row, pl.first * 4u);
        r.b = load_at<uint32_t>(lut_row, pl.second * 4u);
    } else if constexpr (BITS == 8) {   // 512 B: 64 lanes x 8 B
        r.c = load_at<u32x2>(lut_row, (uint32_t)lane * 8u);
    } else if constexpr (BITS == 7) {   // 256 B: 64 lanes x 4 B
        r.a = load_at<uint32_t>(lut_row, (uint32_t)lane * 4u);
    } else {                            // 64 / 128 B: first lanes x 4 B
        if (lane < (1 << BITS) / 2) r.a = load_at<uint32_t>(lut_row, (uint32_t)lane * 4u);
    }
    return r;
}
template <int BITS>
__device__ __forceinline__ TableWords<BITS> lookup_table_fetch(const half_t *lut_row, int lane, const PairLane<BITS> &pl) {
    return lookup_table_fetch<BITS>(scalar_ptr(lut_row), lane, pl);
}

// A point the fetched words cannot be used before.  Put between the loads a kernel issues after the table
// fetch and the staging: otherwise the compiler moves staging arithmetic (a shift of a fetched word) up to
// the fetch, and the wave waits for its table before it has issued its plane loads.
template <int BITS>
__device__ __forceinline__ void lookup_table_arrive(TableWords<BITS> &r) {
    if constexpr (BITS <= 4) asm volatile("" : "+v"(r.a), "+v"(r.b));  // only the words this bit-width fetches
    else if constexpr (BITS == 8) asm volatile("" : "+v"(r.c));
    else asm volatile("" : "+v"(r.a));
}

// Write the fetched table into LDS in the form the lookups expect.
template <int BITS>
__device__ __forceinline__ void lookup_table_stage(const TableWords<BITS> &r, uint8_t *slot, int lane) {
    if constexpr (BITS == 3) {
        reinterpret_cast<uint32_t *>(slot)[lane] = r.a | (r.b << 16);
    } else if constexpr (BITS == 4) {
        u32x4 v;  // (first.lo|hi, second.lo|hi) in entry order 4*lane + {0, 1, 2, 3}
        v[0] = __builtin_amdgcn_perm(r.b, r.a, 0x05040100u);
        v[1] = __builtin_amdgcn_perm(r.b, r.a, 0x07060100u);
        v[2] = __builtin_amdgcn_perm(r.b, r.a, 0x05040302u);
        v[3] = __builtin_amdgcn_perm(r.b, r.a, 0x07060302u);
        reinterpret_cast<u32x4 *>(slot)[lane] = v;
    } else if constexpr (BITS == 8) {
        reinterpret_cast<u32x2 *>(slot)[lane] = r.c;
    } else if constexpr (BITS == 7) {
        reinterpret_cast<uint32_t *>(slot)[lane] = r.a;
    } else {
        if (lane < (1 << BITS) / 2) reinterpret_cast<uint32_t *>(slot)[lane] = r.a;
    }
}

// Workgroup barrier that orders LDS traffic only: outstanding global loads stay in flight across it.
__device__ __forceinline__ void lds_only_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// Activations of WPL consecutive words starting at word wl, as they sit in memory: X[m][wi][j][i] =
// elements (2i, 2i+1) of byte group j of word wl + wi.
template <int M, int WPL>
__device__ __forceinline__ void load_activations_plain(const half_t *__restrict__ x, int K, int wl,
                                                       uint32_t (&X)[M][WPL][4][4]) {
    const global_ptr<const half_t> base = scalar_ptr(x);
#pragma unroll
    for (int m = 0; m < M; m++)
#pragma unroll
        for (int wi = 0; wi < WPL; wi++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                // uniform base + 32-bit byte offset of the lane (M * K * 2 < 2^32)
                const uint32_t byte = ((uint32_t)m * (uint32_t)K + (uint32_t)group_base(wl + wi, j, K)) * 2u;
                const u32x4 v = load_at<u32x4>(base, byte);
#pragma unroll
                for (int i = 0; i < 4; i++) X[m][wi][j][i] = v[i];
            }
}

// Lookup stream over NW words of this lane.  Word n is the plane words q[n][0..BITS), takes its weights
// from LDS table slot[TR(n)] and multiplies the activations X[m][XW(n)]; sums go to acc[TR(n)][m][0..1].
// TR and XW are compile-time maps given as functors returning integral constants.
//
// Pair tables: a lookup costs an LDS round trip of a hundred cycles or more; left to the compiler the
// stream becomes "eight addresses, eight reads, wait, eight uses" and a wave idles through every wait.
// Here it is cut into quads of four lookups, kLookupDepth quads stay in flight (12 reads; the hardware
// counter holds 15), the transpose of the next word is issued while reads return, and scheduling fences
// pin that order (measured 3-7 % faster at 3 bits).  Single tables (5..8 bits) measured faster with the
// compiler's own order, so they are left to it.
constexpr int kLookupDepth = 3;

template <int BITS, int M, int NW, int NT, int XWORDS, typename TR, typename XW>
__device__ __forceinline__ void lookup_dot(const uint32_t (&q)[NW][BITS], const uint8_t (&slot)[NT][LookupTable<BITS>::kBytes],
                                           const uint32_t (&X)[M][XWORDS][4][4], float (&acc)[NT][M][2], TR tr, XW xw) {
    if constexpr (LookupTable<BITS>::kPair) {
        constexpr int QPW = 4, NQ = NW * QPW;   // quad = the four byte groups of one pair register
        uint32_t apair[NW][4];
        uint32_t raw[NQ][4];
        auto issue = [&](auto q_c) {
            constexpr int qd = decltype(q_c)::value, n = qd / QPW, i = qd % QPW;
            constexpr int r = decltype(tr(std::integral_constant<int, n>{}))::value;
            static_for<4>([&](auto c_c) {
                constexpr int c = decltype(c_c)::value;
                const uint32_t off = byte_offset<c, BITS == 4 ? 2 : 0>(apair[n][i]);
                raw[qd][c] = *reinterpret_cast<const uint32_t *>(&slot[r][off]);
            });
        };
        auto consume = [&](auto q_c) {
            constexpr int qd = decltype(q_c)::value, n = qd / QPW, i = qd % QPW;
            constexpr int r = decltype(tr(std::integral_constant<int, n>{}))::value;
            constexpr int wi = decltype(xw(std::integral_constant<int, n>{}))::value;
#pragma unroll
            for (int c = 0; c < 4; c++)
#pragma unroll
                for (int m = 0; m < M; m++) acc[r][m][c & 1] = dot2(raw[qd][c], X[m][wi][3 - c][i], acc[r][m][c & 1]);
        };
        planes_to_adjacent_pairs<BITS>(q[0], apair[0]);
        static_for<(kLookupDepth < NQ ? kLookupDepth : NQ)>([&](auto q_c) { issue(q_c); });
        __builtin_amdgcn_sched_barrier(0);
        static_for<NQ>([&](auto q_c) {
            constexpr int qd = decltype(q_c)::value, ahead = qd + kLookupDepth;
            consume(q_c);
            if constexpr (ahead < NQ) {
                if constexpr (ahead % QPW == 0) planes_to_adjacent_pairs<BITS>(q[ahead / QPW], apair[ahead / QPW]);
                issue(std::integral_constant<int, ahead>{});
            }
            __builtin_amdgcn_sched_barrier(0);
        });
    } else {
        static_for<NW>([&](auto n_c) {
            constexpr int n = decltype(n_c)::value;
            constexpr int r = decltype(tr(n_c))::value;
            constexpr int wi = decltype(xw(n_c))::value;
            uint32_t idx[8];
            planes_to_indices<BITS>(q[n], idx);
            static_for<4>([&](auto i_c) {
                static_for<4>([&](auto c_c) {
                    constexpr int i = decltype(i_c)::value, c = decltype(c_c)::value;
                    const uint32_t o0 = byte_offset<c, 1>(idx[2 * i]);
                    const uint32_t o1 = byte_offset<c, 1>(idx[2 * i + 1]);
                    const uint32_t lo = *reinterpret_cast<const uint16_t *>(&slot[r][o0]);
                    const uint32_t hi = *reinterpret_cast<const uint16_t *>(&slot[r][o1]);
                    const uint32_t w2 = lo | (hi << 16);
#pragma unroll
                    for (int m = 0; m < M; m++) acc[r][m][c & 1] = dot2(w2, X[m][wi][3 - c][i], acc[r][m][c & 1]);
                });
            });
            __builtin_amdgcn_sched_barrier(0);  // one word at a time: interleaving words only costs registers
        });
    }
}

}  // namespace ap

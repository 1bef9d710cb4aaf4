// Fused bitplane dequant -> MFMA GEMM for gfx950, 1 <= M <= 128:
//     out[m,n] = sum_k x[m,k] * lut[n, index_b(n,k)]      (fp16 operands, fp32 accumulate)
//
// The reference has no fused kernel: above 8 activation rows it writes the whole fp16
// weight with dequant_kbit and calls torch.matmul
// (any_precision/modules/AnyPrecisionLinear.py:60-62).  For the batches a serving loop
// sees (tens of rows) that GEMM is bound by reading the fp16 weight it has just written;
// here the planes are read once (w_bits/16 of that traffic) and the dequantised weights
// never leave the register file.
//
// Mapping: v_mfma_f32_16x16x32_f16 wants, in lane l, eight consecutive-k halves of
// B[k][n] for n = l % 16 and k-group l / 16, and the same of A[m][k] for m = l % 16.  The
// packed layout hands out exactly such octets: byte group j of word w of row n holds
// eight consecutive elements, and words 4s..4s+3 of a chunk hold 32 consecutive ones.
// So lane l owns row n0 + l % 16 and word 4s + l / 16; it rebuilds the 32 indices of its
// word, gathers them from its row's table in LDS and has, for every byte group j, one
// B operand ready in registers -- no LDS round trip for the weights.  The matching A
// operand is x[m][k0 + 8 (l/16) .. +7]: 64 contiguous bytes per activation row.
//
// A workgroup is KS waves that share 16 weight rows and split K; their fp32 partial
// tiles meet in LDS and are added in a fixed order.
//
// Plane loads: with VEC4 (K a multiple of 128) a lane loads the four words 16S + 4g .. +3
// of its row in one 16-byte load -- the four lanes of a row cover one 64-byte line -- and
// the words are then transposed across the four 16-lane rows of the wave
// (v_permlane32_swap / v_permlane16_swap) so that lane g holds words 16S + 4i + g,
// i = 0..3: at step i the four lanes of a row again hold four consecutive words.  Without
// VEC4 a lane loads one word per step (16 contiguous bytes per row and instruction) and
// the 64-byte line is re-read from L1/L2 by the next three steps.
#pragma once
#include <type_traits>

#include "ap_bitplane.hpp"
#include "ap_device.hpp"
#include "ap_gemm_launch.hpp"
#include "ap_lookup.hpp"
#include "ap_reciprocal.hpp"

namespace ap {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

constexpr int kGemmRows = 16;     // weight rows per workgroup (one MFMA column block)

// 4x4 transpose of r[0..3] across the four 16-lane rows of the wave: on return r[i] of
// row g holds what r[g] of row i held.
__device__ __forceinline__ void transpose_rows4(uint32_t (&r)[4]) {
    auto a = __builtin_amdgcn_permlane32_swap(r[0], r[2], false, false);  // rows 2,3 of r0 <-> rows 0,1 of r2
    auto b = __builtin_amdgcn_permlane32_swap(r[1], r[3], false, false);
    auto c = __builtin_amdgcn_permlane16_swap(a[0], b[0], false, false);  // odd rows of r0 <-> even rows of r1
    auto d = __builtin_amdgcn_permlane16_swap(a[1], b[1], false, false);
    r[0] = c[0];
    r[1] = c[1];
    r[2] = d[0];
    r[3] = d[1];
}

// MB = activation row blocks of 16 (M <= 16*MB).  RB = blocks of 16 weight rows a wave works on in
// lockstep: every activation operand it loads then feeds RB matrix instructions instead of one,
// which divides the L2 traffic of the activations by RB -- at the price of 1/RB as many
// workgroups, so only linears with many rows use RB = 2.  Grid: ceil(N / (16 RB)) workgroups of (64, KS).
// LOOKAHEAD: see the step below.
template <int BITS, int MB, bool VEC4, int MP, int RB, bool LOOKAHEAD = false>
__global__ __launch_bounds__(kGemmMaxSplit *kWave) void gemm_kbit_kernel(
    const half_t *__restrict__ x, const uint32_t *__restrict__ qweight, const half_t *__restrict__ lut,
    half_t *__restrict__ out, int M, int N, int K, int KS, uint32_t ks_magic) {
    constexpr int NC = 1 << BITS;
    constexpr int WPS = VEC4 ? 4 : 1;             // words per lane and step
    constexpr int ROWS = kGemmRows * RB;    // weight rows per workgroup
    // 3 and 4 bits: a table of the weights of two ADJACENT elements per row (ap_lookup.hpp) -- one ds_read_b32 per
    // half2 of a B operand, and a quarter of the bit operations of the single-index form.
    constexpr bool PAIR = LookupTable<BITS>::kPair;
    constexpr int TB = LookupTable<BITS>::kBytes;  // bytes of one row's table in LDS
    constexpr int TQ = ROWS * NC / 8;       // 16-byte quads of the rows' tables in global memory
    __shared__ __attribute__((aligned(16))) uint8_t tables[ROWS][TB];
    // One private region per wave.  While the wave computes it stages activations there: MP rows x 16
    // octets (4 byte groups x 4 words).  Afterwards the same bytes carry the wave's partial tiles
    // (RB x MB x 4 x 64 floats) to the combine step -- LDS operations of one wave complete in order, so
    // the wave's last operand reads are done before its tile is written.
    constexpr int XS = MP * 16 > RB * MB * 64 ? MP * 16 : RB * MB * 64;
    __shared__ u32x4 xs[kGemmMaxSplit][XS];
    static_assert(MP == 0 || (MP >= 8 && MP <= 16 * MB && (MP & (MP - 1)) == 0), "");

    // every argument in scalar registers by one clause of scalar loads and one wait (the compiler alone loads
    // an argument where it is first used: a dependent round trip to the scalar cache each)
    asm volatile("" : "+s"(x), "+s"(qweight), "+s"(lut), "+s"(out), "+s"(M), "+s"(N), "+s"(K), "+s"(KS), "+s"(ks_magic));
    const int lane = threadIdx.x;
    const int ks = __builtin_amdgcn_readfirstlane(threadIdx.y);  // KS = blockDim.y, passed as an argument
    const int col = lane & 15, grp = lane >> 4;
    const int W = K >> 5;
    const size_t plane_bytes = (size_t)N * W * sizeof(uint32_t);  // below 2^32 (the host checks)
    const int n0 = blockIdx.x * ROWS;

    // this wave's range of steps (4 * WPS words of every row per step): steps * ks / KS by a multiplication
    // with ks_magic = reciprocal_ceil(KS) from the host (ap_reciprocal.hpp), exact for steps * (ks + 1) < 2^29
    // (KS <= 8, K < 2^33)
    const int steps = (W + 4 * WPS - 1) / (4 * WPS);
    auto over_ks = [&](int n) { return (int)div_by_reciprocal_ceil((uint32_t)n, (uint32_t)KS, ks_magic); };
    const int s_begin = over_ks(steps * ks), s_end = over_ks(steps * (ks + 1));

    // byte offset of this lane's row inside a plane (rows past N repeat row N-1 and are not stored); a plane
    // word is loaded from the scalar plane base plus this offset plus the word's
    const global_ptr<const char> qbytes = scalar_ptr(reinterpret_cast<const char *>(qweight));
    const global_ptr<const half_t> xg = scalar_ptr(x);
    uint32_t row_off[RB];
#pragma unroll
    for (int rb = 0; rb < RB; rb++)
        row_off[rb] = (uint32_t)min(n0 + rb * kGemmRows + col, N - 1) * (uint32_t)W * (uint32_t)sizeof(uint32_t);
    // q[rb][p][i]: row block rb, plane p, i-th word of this lane for the step
    auto fetch = [&](int step, uint32_t(&q)[RB][BITS][WPS]) {
        if constexpr (VEC4) {
            // W % 4 == 0: a quad is entirely inside the row or entirely past its end (then it is
            // clamped to the last quad and never used)
            const int w = min(16 * step + 4 * grp, W - 4);
#pragma unroll
            for (int rb = 0; rb < RB; rb++)
#pragma unroll
                for (int p = 0; p < BITS; p++) {
                    const u32x4 v = load_at_nt<u32x4>(scalar_ptr(qbytes + p * plane_bytes), row_off[rb] + (uint32_t)w * 4u);
#pragma unroll
                    for (int i = 0; i < 4; i++) q[rb][p][i] = v[i];
                }
        } else {
            // plain (temporal) loads: the 64-byte line is needed again by the next three steps
            const int w = min(4 * step + grp, W - 1);
#pragma unroll
            for (int rb = 0; rb < RB; rb++)
#pragma unroll
                for (int p = 0; p < BITS; p++)
                    q[rb][p][0] = load_at<uint32_t>(scalar_ptr(qbytes + p * plane_bytes), row_off[rb] + (uint32_t)w * 4u);
        }
    };

    // byte offset of this lane's activation row in each row block (rows past M repeat row M-1)
    uint32_t xoff[MB];
#pragma unroll
    for (int mb = 0; mb < MB; mb++) xoff[mb] = (uint32_t)min(mb * 16 + col, M - 1) * (uint32_t)K * 2u;
    const int full_chunks = W >> 5;                // chunks of 32 words; a shorter one may follow
    const uint32_t tail_stride = (uint32_t)(W & 31) * 16u;  // bytes of x between byte groups in the tail chunk
    // x byte offset (within a row) of byte group j of the wi-th word of this lane in `step`; a word past the row
    // end takes the last word's
    auto a_offset = [&](int step, int wi, int j) {
        const int w = min(4 * (WPS * step + wi) + grp, W - 1);
        const int chunk = w >> 5;
        return ((uint32_t)chunk << 11) + ((uint32_t)(w & 31) << 4) + (uint32_t)j * (chunk == full_chunks ? tail_stride : 512u);
    };
    // The unit of the inner schedule is the octet (one byte group of one word: one B operand,
    // MB MFMAs).  Its A operand is 16 bytes of x per lane, lane (m, g) taking row m and the
    // g-th octet of a 64-byte run.  Every workgroup reads its K-slices of ALL of x, so the
    // activations are re-read N/16 times from L2 -- (N/16) * M * K * 2 bytes, more than the
    // planes from M = 2 * w_bits rows on.
    // MP == 0: the operands are loaded straight from global memory, AHEAD octets early.  (Requesting all sixteen
    // of a step at once, with the planes or right after the tables, measured slower: so many loads whose lanes
    // sit in sixteen different rows delay the plane data that every wave waits for first.)
    // MP > 0: the wave loads the x block of a word group (MP rows x 4 runs of 64 bytes) with
    // adjacent lanes on adjacent addresses, parks it in its own LDS region and reads the
    // operands from there (slots skewed by the octet index so that writes and reads are free
    // of bank conflicts; LDS operations of one wave complete in order, so no barrier).
    constexpr int OCT = 4 * WPS;
    constexpr int AHEAD = MB == 1 ? 4 : (MB == 2 ? 2 : 1);
    constexpr int NL = MP / 4;  // staging loads per lane and word group

    // Load order: planes of the first step, then the tables -- both in flight
    // together, and the tables are staged while nothing else could run anyway.  The tables of the
    // workgroup's rows are contiguous in lut (rows past N re-read the last 16 bytes of the
    // array; their columns are never stored).
    // (every wave has at least one step: the host launches at most as many waves as there are steps)
    uint32_t qa[RB][BITS][WPS], qb[RB][BITS][WPS];
    fetch(s_begin, qa);
    if constexpr (PAIR) {
        // wave ks builds the pair tables of rows ks, ks + KS, ...: the loads of the first ROWS / 8 of them (all,
        // when the workgroup has its eight waves) are issued together
        constexpr int NT = ROWS / kGemmMaxSplit;
        const PairLane<BITS> pl = pair_lane<BITS>(lane);
        TableWords<BITS> tw[NT];
#pragma unroll
        for (int i = 0; i < NT; i++) {
            const int r = min(ks + i * KS, ROWS - 1);
            tw[i] = lookup_table_fetch<BITS>(lut + (size_t)min(n0 + r, N - 1) * NC, lane, pl);
        }
#pragma unroll
        for (int i = 0; i < NT; i++)
            if (ks + i * KS < ROWS) lookup_table_stage<BITS>(tw[i], &tables[ks + i * KS][0], lane);
        for (int r = ks + NT * KS; r < ROWS; r += KS)
            lookup_table_stage<BITS>(lookup_table_fetch<BITS>(lut + (size_t)min(n0 + r, N - 1) * NC, lane, pl), &tables[r][0], lane);
    } else {
        const int nthr = KS * kWave;
        const global_ptr<const u32x4> src = (global_ptr<const u32x4>)reinterpret_cast<uint64_t>(lut);
        u32x4 *dst = reinterpret_cast<u32x4 *>(&tables[0][0]);
        const long long first = (long long)n0 * (NC / 8), last = (long long)N * (NC / 8) - 1;
        for (int i = ks * kWave + lane; i < TQ; i += nthr) dst[i] = src[min(first + i, last)];
    }
    __syncthreads();
    // LDS byte address of this lane's table (LDS pointers are 32-bit offsets)
    typedef __attribute__((address_space(3))) half_t lds_half_t;
    typedef __attribute__((address_space(3))) uint32_t lds_u32_t;
    const uint32_t tab_base0 = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) uint8_t *)&tables[0][0]) + (uint32_t)col * TB;

    float4_t acc[RB][MB];
#pragma unroll
    for (int rb = 0; rb < RB; rb++)
#pragma unroll
        for (int mb = 0; mb < MB; mb++) acc[rb][mb] = float4_t{0.f, 0.f, 0.f, 0.f};

    // One step: transpose the planes of each word to indices, gather, multiply.  CHECK: the
    // step may reach past the end of the row (only the last step of a row can).
    // LOOKAHEAD: the lookups run one word ahead of the matrix instructions -- the 16 (pair tables) or 32 gathers
    // of word wi + 1 are issued before the four octets of word wi are multiplied (a second set of B operands), so
    // the wave waits for LDS once per word and not once per octet.  Measured 2-9 % faster where a CU holds one
    // workgroup (linears of up to 16 rows per CU), and 5-20 % slower where it holds several, whose waves cover
    // each other's waits and lose occupancy to the extra registers: the host chooses.
    auto process = [&](auto check_c, int step, uint32_t(&q)[RB][BITS][WPS]) {
        constexpr bool CHECK = decltype(check_c)::value;
        bool live[WPS];
#pragma unroll
        for (int wi = 0; wi < WPS; wi++) live[wi] = !CHECK || 4 * (WPS * step + wi) + grp < W;  // words past the row end contribute zeros

        // ---- direct path (MP == 0): fragments from global memory, AHEAD octets early
        half8_t a[MP == 0 ? OCT : 1][MB];
        auto load_a = [&](auto t_c) {
            constexpr int t = decltype(t_c)::value;
            if constexpr (MP == 0 && t < OCT) {
                const uint32_t koff = a_offset(step, t / 4, t % 4);
#pragma unroll
                for (int mb = 0; mb < MB; mb++)
                    a[t][mb] = load_at<half8_t>(xg, xoff[mb] + koff);
            }
        };
        // ---- staged path (MP > 0): lane = (row r + 4 i, byte group sj, octet sg of the run)
        const int sg = lane & 3, sj = (lane >> 2) & 3, sr = lane >> 4;
        u32x4 xr[NL > 0 ? NL : 1];
        auto stage_load = [&](int wi) {
            if constexpr (MP > 0) {
                int w = 4 * (WPS * step + wi) + sg;
                if (CHECK) w = min(w, W - 1);
                const int chunk = w >> 5;
                const uint32_t koff = ((uint32_t)chunk << 11) + ((uint32_t)(w & 31) << 4) +
                                      (uint32_t)sj * (chunk == full_chunks ? tail_stride : 512u);
#pragma unroll
                for (int i = 0; i < NL; i++) {
                    const uint32_t roff = (uint32_t)min(sr + 4 * i, M - 1) * (uint32_t)K * 2u;
                    xr[i] = load_at<u32x4>(xg, roff + koff);
                }
            }
        };
        auto stage_store = [&]() {
            if constexpr (MP > 0) {
                const int o = 4 * sj + sg;
#pragma unroll
                for (int i = 0; i < NL; i++) xs[ks][o * MP + ((sr + 4 * i + o) & (MP - 1))] = xr[i];
                __builtin_amdgcn_wave_barrier();
            }
        };

        // B operands in flight: bws[slot][j][rb] = the eight weights of byte group j (LOOKAHEAD: slot = word & 1)
        u32x4 bws[LOOKAHEAD ? 2 : 1][LOOKAHEAD ? 4 : 1][RB];
        // index bytes hold the byte offset into the table (index * 2) where that fits a byte
        constexpr int PRE = BITS <= 7 ? 1 : 0;
        uint32_t idx[LOOKAHEAD ? 2 : 1][RB][PAIR ? 4 : 8];
        auto indices = [&](auto wi_c) {
            constexpr int wi = decltype(wi_c)::value, slot = LOOKAHEAD ? wi & 1 : 0;
#pragma unroll
            for (int rb = 0; rb < RB; rb++) {
                uint32_t qq[BITS];
#pragma unroll
                for (int p = 0; p < BITS; p++) qq[p] = q[rb][p][wi];
                if constexpr (PAIR) planes_to_adjacent_pairs<BITS>(qq, idx[slot][rb]);
                else planes_to_indices<BITS, PRE>(qq, idx[slot][rb]);
            }
        };
        auto gather = [&](auto wi_c, auto j_c) {
            constexpr int wi = decltype(wi_c)::value, j = decltype(j_c)::value, c = 3 - j, slot = LOOKAHEAD ? wi & 1 : 0;
            static_for<RB>([&](auto rb_c) {
                constexpr int rb = decltype(rb_c)::value;
                const uint32_t tab_base = tab_base0 + rb * (kGemmRows * TB);
                static_for<4>([&](auto e_c) {
                    constexpr int i = decltype(e_c)::value;
                    uint32_t packed;
                    if constexpr (PAIR) {
                        // byte c of idx[i]: the entry of elements (2i, 2i+1) of byte group j -- at 3 bits already its byte offset
                        uint32_t a0;
                        if constexpr (BITS == 3) a0 = byte_add<c>(tab_base, idx[slot][rb][i]);
                        else a0 = tab_base + byte_offset<c, 2>(idx[slot][rb][i]);
                        packed = *reinterpret_cast<const lds_u32_t *>(a0);
                    } else {
                        uint32_t a0, a1;
                        if constexpr (PRE) {
                            a0 = byte_add<c>(tab_base, idx[slot][rb][2 * i]);
                            a1 = byte_add<c>(tab_base, idx[slot][rb][2 * i + 1]);
                        } else {
                            a0 = tab_base + byte_offset<c, 1>(idx[slot][rb][2 * i]);
                            a1 = tab_base + byte_offset<c, 1>(idx[slot][rb][2 * i + 1]);
                        }
                        half2_t h;
                        h.x = *reinterpret_cast<const lds_half_t *>(a0);
                        h.y = *reinterpret_cast<const lds_half_t *>(a1);
                        packed = __builtin_bit_cast(uint32_t, h);
                    }
                    bws[slot][LOOKAHEAD ? j : 0][rb][i] = live[wi] ? packed : 0u;
                });
            });
        };
        auto lookups = [&](auto wi_c) {  // a whole word
            indices(wi_c);
            static_for<4>([&](auto j_c) { gather(wi_c, j_c); });
        };

        if constexpr (MP > 0) stage_load(0);
        static_for<AHEAD>([&](auto t_c) { load_a(t_c); });
        if constexpr (VEC4) {
#pragma unroll
            for (int rb = 0; rb < RB; rb++)
#pragma unroll
                for (int p = 0; p < BITS; p++) transpose_rows4(q[rb][p]);
        }
        if constexpr (LOOKAHEAD) lookups(std::integral_constant<int, 0>{});
        static_for<WPS>([&](auto wi_c) {
            constexpr int wi = decltype(wi_c)::value;
            if constexpr (MP > 0) {
                stage_store();
                if constexpr (wi + 1 < WPS) stage_load(wi + 1);
            }
            if constexpr (!LOOKAHEAD) indices(wi_c);
            else if constexpr (wi + 1 < WPS) lookups(std::integral_constant<int, wi + 1>{});
            if constexpr (LOOKAHEAD) __builtin_amdgcn_sched_barrier(0);  // keeps the gathers of word wi + 1 ahead of the multiplications of word wi
            static_for<4>([&](auto j_c) {
                constexpr int j = decltype(j_c)::value, t = 4 * wi + j;
                load_a(std::integral_constant<int, t + AHEAD>{});
                if constexpr (!LOOKAHEAD) gather(wi_c, j_c);
#pragma unroll
                for (int mb = 0; mb < MB; mb++) {
                    half8_t afrag;
                    if constexpr (MP > 0) {
                        const int o = 4 * j + grp;
                        const int m = (mb * 16 + col) & (MP - 1);  // MP < 16: rows repeat, their results are not stored
                        afrag = __builtin_bit_cast(half8_t, xs[ks][o * MP + ((m + o) & (MP - 1))]);
                    } else {
                        afrag = a[t][mb];
                    }
                    // words past the row end: zero activations as well as zero weights (0 * inf would be NaN)
                    if constexpr (CHECK) {
                        if (!live[wi]) afrag = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
                    }
#pragma unroll
                    for (int rb = 0; rb < RB; rb++)
                        acc[rb][mb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(afrag, __builtin_bit_cast(half8_t, bws[LOOKAHEAD ? wi & 1 : 0][LOOKAHEAD ? j : 0][rb]),
                                                                             acc[rb][mb], 0, 0, 0);
                }
            });
        });
    };

    auto run = [&](int step, uint32_t(&q)[RB][BITS][WPS]) {
        if (4 * WPS * (step + 1) <= W)
            process(std::false_type{}, step, q);
        else
            process(std::true_type{}, step, q);
    };
    // With few planes the next step's words are fetched while this step computes, two register sets taking turns
    // (the loop body is written out twice: handing the prefetched registers over with copies makes the wave wait
    // for those loads where the copies stand); with many, the second set is not worth its registers (no
    // measurable gain) and a step's words are fetched when the step before it is done.
    constexpr bool PREFETCH = RB * BITS * WPS <= 20;
    int step = s_begin;
    if constexpr (PREFETCH) {
        for (;;) {
            if (step + 1 < s_end) fetch(step + 1, qb);
            run(step, qa);
            if (++step >= s_end) break;
            if (step + 1 < s_end) fetch(step + 1, qa);
            run(step, qb);
            if (++step >= s_end) break;
        }
    } else {
        for (;;) {
            run(step, qa);
            if (++step >= s_end) break;
            fetch(step, qa);
        }
    }

    // Combine the K-split partial tiles in wave order (also with one wave: it keeps the
    // accumulator indices static).  D[i][j]: lane l holds rows i = 4 (l / 16) + v, column l % 16.
    const global_ptr<half_t> out_g = (global_ptr<half_t>)reinterpret_cast<uint64_t>(out);  // a global store, not a flat one
    float *mine = reinterpret_cast<float *>(&xs[ks][0]);
#pragma unroll
    for (int rb = 0; rb < RB; rb++)
#pragma unroll
        for (int mb = 0; mb < MB; mb++)
#pragma unroll
            for (int v = 0; v < 4; v++) mine[((rb * MB + mb) * 4 + v) * kWave + lane] = acc[rb][mb][v];
    __syncthreads();
    for (int t = ks; t < RB * MB * 4; t += KS) {
        const int rb = t / (MB * 4), mb = (t >> 2) % MB, v = t & 3;
        float sum = 0.f;
        for (int kk = 0; kk < KS; kk++) sum += reinterpret_cast<const float *>(&xs[kk][0])[t * kWave + lane];
        const int m = mb * 16 + 4 * grp + v, n = n0 + rb * kGemmRows + col;
        if (m < M && n < N) out_g[(size_t)m * N + n] = (half_t)sum;
    }
}

}  // namespace ap

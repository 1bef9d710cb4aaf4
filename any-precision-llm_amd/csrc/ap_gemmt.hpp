// Tiled fused bitplane dequant -> MFMA GEMM for gfx950, for batches of tens to hundreds of activation rows:
//     out[m,n] = sum_k x[m,k] * lut[n, index_b(n,k)]      (fp16 operands, fp32 accumulate)
//
// The reference writes the whole fp16 weight with dequant_kbit and calls torch.matmul above 8 rows
// (any_precision/modules/AnyPrecisionLinear.py:60-62).  The K-split kernel of ap_gemm.hpp keeps the weights in
// registers but re-reads the activations from L2 once per 16 weight rows, which bounds it from about 64 rows on.
// Here a workgroup owns a tile of BN = 64 RB weight rows x BM = 16 MBW activation rows for the WHOLE of K:
//   * four waves, each on its own 16 RB weight rows; a wave rebuilds its weights in registers exactly as ap_gemm.hpp
//     does (lane = row l % 16 and word 4s + l / 16; one B operand per byte group of a word) -- no LDS round trip and
//     one table lookup per weight and tile of activation rows;
//   * the activations of the tile are staged ONCE per workgroup in LDS, in two or four buffers, 256 contiguous bytes
//     per row and stage (byte group j of the 16 words of a step: 128 consecutive elements), and every A operand a wave
//     reads from there feeds RB matrix instructions; the 16-byte units of a row are XOR-swizzled with the row number so
//     that the 16 rows of an operand read hit 16 different bank groups.  While a stage is in work the next one (or
//     the third next) is brought in by direct global -> LDS loads (no registers, no LDS store instructions); units
//     past the end of a row are fetched from an array of zeros;
//   * the lookup tables sit in LDS by entry and slot where that fits, so that the lanes served together read
//     different banks (below);
//   * accumulators (RB x MBW tiles of 16 x 16) stay in registers over the whole K loop: no K-split, no combine.
// Per stage a wave issues 4 x RB x MBW matrix instructions between two barriers.  K must be a multiple of 128.
// MBW = 1 and 2 (tiles of 16 and 32 activation rows) are for grids that would leave CUs idle: the same weights are then
// dequantised by several workgroups, each for fewer activation rows.
// One launch serves up to four linears that share x (q/k/v, gate/up): their tiles of 64 weight rows are numbered through
// (GemmtMembers), which fills the chip where one linear alone leaves CUs idle.
#pragma once
#include <type_traits>

#include "ap_bitplane.hpp"
#include "ap_device.hpp"
#include "ap_gemm.hpp"
#include "ap_gemmt_launch.hpp"
#include "ap_lookup.hpp"
#include "ap_reciprocal.hpp"

namespace ap {

// What a direct load fetches for a 16-byte unit that lies past the end of its row (or belongs to an idle iteration).
__device__ const uint32_t kGemmtZeros[64] = {};

// KH = 1 or 2 groups of four waves per workgroup; with 2, group kh walks half of K (steps kh * ceil(steps / 2) ..) on its
// own stage buffers and the two partial tiles are added in LDS at the end (group 0's sum + group 1's, always in that
// order).  Twice the waves per tile: for grids that leave CUs with one workgroup of four waves, where no pipe is busy
// and waves wait for each other's LDS round trips.
template <int BITS, int RB, int MBW, int KH>
__global__ __launch_bounds__(kGemmtWaves *kWave *KH) void gemmt_kbit_kernel(const half_t *__restrict__ x, const GemmtMembers mem,
                                                                             int M, int K, int grid_m, uint32_t tile_div,
                                                                             uint32_t tile_magic) {
    constexpr int NC = 1 << BITS;
    // 3 bits: the table of the weights of two adjacent elements (ap_lookup.hpp; 64 dword entries per row): half the table
    // reads, which are what loads the LDS port.  At 4 bits that table is 1 KB per row, 64 KB per workgroup: it pays where a CU
    // holds one workgroup anyway (the grids that run two K halves: 4096 x 4096 at 128 rows 26 us against 31) and costs
    // where it halves the workgroups per CU (11008 x 4096 at 256 rows: 92 us against 74), so only KH = 2 uses it.
    constexpr bool PAIR = BITS == 3 || (BITS == 4 && KH == 2);
    constexpr int TB = PAIR ? LookupTable<BITS>::kBytes : 2 * NC;  // bytes of one row's table in LDS
    constexpr int WROWS = kGemmRows * RB;                           // weight rows per wave
    constexpr int BN = kGemmtWaves * WROWS, BM = 16 * MBW;
    constexpr int NTHR = kGemmtWaves * kWave;
    __shared__ __attribute__((aligned(16))) uint8_t tables[BN][TB];
    // Tables laid out by entry and slot, [wave][entry][slot] dwords: a table read is one random entry per lane, and with a
    // table per row 32 random addresses cost the LDS about 3.5 cycles instead of 1.  Here the 32 lanes it serves per
    // cycle -- 16 rows x 2 -- read by slot.  Two-half form (a CU to itself, LDS to spare): slot = 16 (lane / 16 & 1) +
    // row, two copies of every row's table, 32 different banks whatever the entries.  One group of waves per tile
    // (two or three workgroups share a CU): slot = row, one copy, the two lanes of a row collide when their entries
    // differ (2 cycles), in the LDS a table per row would take or little more.
    //   3 bits: the 64-entry pair table (8 or 4 KB per wave);
    //   4 bits: two-half form the 256-entry pair table, one copy (the same 64 KB as a table per row); else the plain
    //           table as below;
    //   4..8 bits: the plain table with one fp16 entry per dword; two copies up to 7 bits in the two-half form
    //           (16..64 KB per workgroup), one copy at 8 bits (64 KB) and with one group of waves (up to 6 bits there:
    //           1..16 KB; the tables of 7 and 8 bits would cost a workgroup per CU -- except the 128-row tile at 8
    //           bits, which has its CU to itself already).
    constexpr bool CF = BITS == 3 && RB == 1;
    constexpr bool CF4 = BITS == 4 && RB == 1 && KH == 2;
    constexpr bool CF16 = !PAIR && RB == 1 && (KH == 2 || BITS <= 6 || (BITS == 8 && MBW == 8));
    constexpr int SLOTS = (KH == 1 || BITS == 8) ? 16 : 32;
    constexpr int ESHIFT = SLOTS == 32 ? 7 : 6;  // log2 of the bytes of an entry
    __shared__ uint32_t cftab[CF ? kGemmtWaves * 64 * SLOTS : (CF4 ? kGemmtWaves * 256 * 16 : (CF16 ? kGemmtWaves * NC * SLOTS : 1))];
    // The stage buffers, [K half][activation row][16-byte unit ^ (row & 15)] each: separate arrays, so that the
    // compiler can tell the buffer a direct load fills from the one the matrix operands are read from (it waits for
    // every outstanding direct load before an LDS read that may touch its destination).  Stage t of a group lives in
    // buffer t % NBUF and is requested PD = NBUF - 1 stages before it is used: one stage ahead for tiles of 64 and 128
    // rows, whose stages are long enough to cover the load, three for the narrow tiles (a stage of a 16-row tile is
    // about 150 instructions per wave and used to wait for its successor's load every time).
    constexpr int NBUF = MBW <= 2 ? 4 : 2, PD = NBUF - 1;
    __shared__ u32x4 xt0[KH][BM][16], xt1[KH][BM][16];
    __shared__ u32x4 xt2[NBUF == 4 ? KH : 1][NBUF == 4 ? BM : 1][16], xt3[NBUF == 4 ? KH : 1][NBUF == 4 ? BM : 1][16];
    static_assert(KH == 1 || KH == 2, "");
    static_assert(BN == 64, "the host numbers tiles of 64 weight rows through the members (GemmtMembers::tile0)");
    static_assert(KH == 1 || RB * MBW * 4 * kWave * kGemmtWaves * 4 <= (int)sizeof(xt0) / KH, "partial tiles fit a half's stage buffer");

    const int lane = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.y);
    const int wv = wave % kGemmtWaves, kh = wave / kGemmtWaves;  // row group of the wave, its half of K
    const int tid = wv * kWave + lane;                            // thread within the half
    const int col = lane & 15, grp = lane >> 4;
    // Member 0 (the only one of a plain call) and the scalars every workgroup needs, named in ONE empty statement that
    // wants them in scalar registers: one clause of scalar loads and one wait fetch them (the compiler alone loads an
    // argument where it is first used -- here a chain of five dependent round trips to the scalar cache before the
    // first plane load).  Pointers travel through it as integers and get their address space back afterwards.
    static_assert(kGemmtMaxGroup == 4, "the member selection below is written out for four");
    uint64_t x_i = reinterpret_cast<uint64_t>(x), q_i = reinterpret_cast<uint64_t>(mem.qweight[0]),
             lut_i = reinterpret_cast<uint64_t>(mem.lut[0]), out_i = reinterpret_cast<uint64_t>(mem.out[0]);
    int N0 = mem.N[0], count = mem.count, t1 = mem.tile0[1], t2 = mem.tile0[2], t3 = mem.tile0[3], t4 = mem.tile0[4];
    long long ldo0 = mem.ldo[0];
    asm volatile("" : "+s"(x_i), "+s"(q_i), "+s"(lut_i), "+s"(out_i), "+s"(N0), "+s"(count), "+s"(t1), "+s"(t2), "+s"(t3),
                      "+s"(t4), "+s"(ldo0), "+s"(M), "+s"(K), "+s"(grid_m), "+s"(tile_div), "+s"(tile_magic));
    const int W = K >> 5;
    // Workgroup -> tile.  Consecutive workgroups go round-robin to the 8 XCDs, each with its own L2, and the tiles of
    // one block of weight rows over the activation rows read the same planes: they get workgroup numbers 8 apart, so
    // that they run on one XCD at about the same time and the planes come from HBM once.  Workgroup id = 8 (grid_m a +
    // m) + c stands for weight-row tile 8 a + c and activation-row tile m (the grid is padded to whole groups of 8).
    // Beyond 8 tiles of activation rows the activations are the larger stream (16384 rows: 128 MB against 17 MB of
    // planes at 3 bits): there the weight-row tiles run fastest, so that the workgroups in flight share one tile of
    // activation rows in L2 (the other order measured 0.45 PFLOP/s against 0.70 there).
    const int tiles = count <= 1 ? t1 : (count == 2 ? t2 : (count == 3 ? t3 : t4));  // tile0[count]
    // grid_m = ceil(M / BM) and tile_div = 8 grid_m (up to 8 tiles of activation rows) or the padded number of
    // weight-row tiles come from the host with tile_magic = reciprocal_floor(tile_div) (ap_reciprocal.hpp): the
    // workgroup number is divided by one multiplication and a correction step.
    uint32_t wq, wr;
    divmod_by_reciprocal(blockIdx.x, tile_div, tile_magic, wq, wr);
    int tile_n, tile_m;
    if (grid_m <= 8) {
        tile_n = 8 * (int)wq + (int)(wr & 7u);
        tile_m = (int)(wr >> 3);
    } else {
        tile_n = (int)wr;
        tile_m = (int)wq;
    }
    if (tile_n >= tiles) return;  // padding (workgroup-uniform)
    // the linear this tile belongs to (workgroup-uniform) and the tile's place in it; a launch of several linears
    // reads its member's fields by index (one more clause of scalar loads; a plain call skips it)
    int N = N0, first_tile = 0;
    long long ldo = ldo0;
    if (count > 1) {
        int g = tile_n >= t1 ? 1 : 0;  // tile0 ascends
        g = (count > 2 && tile_n >= t2) ? 2 : g;
        g = (count > 3 && tile_n >= t3) ? 3 : g;
        if (g > 0) {
            q_i = reinterpret_cast<uint64_t>(mem.qweight[g]);
            lut_i = reinterpret_cast<uint64_t>(mem.lut[g]);
            out_i = reinterpret_cast<uint64_t>(mem.out[g]);
            N = mem.N[g];
            ldo = mem.ldo[g];
            first_tile = g == 1 ? t1 : (g == 2 ? t2 : t3);
        }
    }
    x = (const half_t *)(global_ptr<const half_t>)x_i;
    const uint32_t *__restrict__ qweight = (const uint32_t *)(global_ptr<const uint32_t>)q_i;
    const half_t *__restrict__ lut = (const half_t *)(global_ptr<const half_t>)lut_i;
    half_t *__restrict__ out = (half_t *)(global_ptr<half_t>)out_i;
    const int nb = (tile_n - first_tile) * BN;  // first weight row of the workgroup
    const size_t plane_stride = (size_t)N * W;
    const int n0 = nb + wv * WROWS;     // ... of this wave
    const int m0 = tile_m * BM;         // first activation row of the tile
    const int steps = (W + 15) >> 4;    // 16 words of every row per step
    const int nit = (steps + KH - 1) / KH;   // steps per K half; a half with one step fewer idles through the last
    // (all workgroups walk K in the same order: those in flight then read the same columns of the activations at
    // about the same time and share them in L2 -- walking from staggered starting steps measured 10-35 % slower)
    // Iteration i of this half: its step, clamped into the row (an idle iteration loads valid plane words and uses none).
    auto step_at = [&](int i) { return min(kh * nit + i, steps - 1); };
    auto active_at = [&](int i) { return kh * nit + i < steps; };

    const uint32_t *wrow[RB];  // rows past N repeat row N-1 and are not stored
#pragma unroll
    for (int rb = 0; rb < RB; rb++) wrow[rb] = qweight + (size_t)min(n0 + rb * kGemmRows + col, N - 1) * W;
    // one 16-byte load per plane: the four words 16 step + 4 grp .. + 3 (W % 4 == 0: a quad lies inside the row or
    // past its end; then it is clamped to the last quad and never used)
    auto fetch = [&](int step, uint32_t(&q)[RB][BITS][4]) {
        const int w = min(16 * step + 4 * grp, W - 4);
#pragma unroll
        for (int rb = 0; rb < RB; rb++)
#pragma unroll
            for (int p = 0; p < BITS; p++) {
                const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(wrow[rb] + p * plane_stride + w));
#pragma unroll
                for (int i = 0; i < 4; i++) q[rb][p][i] = v[i];
            }
    };

    // ---- activation stages: thread = (unit su of the 256-byte run, row sr + 16 i)
    const int su = tid & 15, sr = tid >> 4;
    const int full_chunks = W >> 5;
    const uint32_t tail_stride = (uint32_t)(W & 31) * 16u;  // bytes of x between byte groups in the tail chunk
    uint32_t xrow[MBW];                                     // byte offset of this thread's activation rows (past M: row M-1)
#pragma unroll
    for (int i = 0; i < MBW; i++) xrow[i] = (uint32_t)min(m0 + sr + 16 * i, M - 1) * (uint32_t)K * 2u;
    auto stage_buffer = [&](auto buf_c) -> auto & {
        constexpr int buf = decltype(buf_c)::value;
        if constexpr (buf == 0) return xt0;
        else if constexpr (buf == 1) return xt1;
        else if constexpr (buf == 2) return xt2;
        else return xt3;
    };

    // A stage goes straight from global memory into LDS (no registers, no LDS store instruction): lane l of a wave
    // writes the l-th 16-byte slot of the 1 KB that holds the wave's four rows, so it requests the unit that belongs
    // there (slot = unit ^ row).  CHECK: the stage may have units of words past the end of the row, or belong to an
    // iteration past the group's share of K; those units come from an array of zeros instead (nothing can be zeroed
    // on the way).
    const char *const zeros = reinterpret_cast<const char *>(kGemmtZeros) + 16 * su;
    auto stage_dma = [&](auto check_c, int it_idx, int j, auto buf_c) {
        auto &xt = stage_buffer(buf_c);
        const int s = kh * nit + it_idx;  // the step, not clamped
        const int w0 = 16 * s, chunk = w0 >> 5, u = su ^ sr;
        const bool valid = !decltype(check_c)::value || (it_idx < nit && w0 + u < W);
        const uint32_t koff = ((uint32_t)chunk << 11) + ((uint32_t)((w0 & 31) + u) << 4) +
                              (uint32_t)j * (chunk == full_chunks ? tail_stride : 512u);
#pragma unroll
        for (int i = 0; i < MBW; i++) {
            const char *src = valid ? reinterpret_cast<const char *>(x) + (size_t)(xrow[i] + koff) : zeros;
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)src,
                                             (__attribute__((address_space(3))) void *)&xt[kh][16 * i + 4 * wv][0], 16, 0, 0);
        }
    };

    // ---- prologue: planes of step 0, the first PD stages, tables
    uint32_t q[RB][BITS][4];
    fetch(step_at(0), q);
    static_for<PD>([&](auto t_c) {
        constexpr int t = decltype(t_c)::value;
        stage_dma(std::true_type{}, 0, t, std::integral_constant<int, t % NBUF>{});
    });
    if constexpr (CF) {
        // entry e = (f2 s2 f1 s1 f0 s0) holds (lut[f], lut[s]).  lane = (row, copy, f2) and the group of waves is s2 with two
        // K halves, lane = (row, s2, f2) with one: a lane writes the 16 entries (f1 s1 f0 s0) of its quarter of the table
        // from the halves of its row's eight values.
        const int f2 = lane >> 5, s2 = KH == 2 ? kh : (lane >> 4) & 1;
        const u32x4 t = *reinterpret_cast<const u32x4 *>(lut + (size_t)min(n0 + (lane & 15), N - 1) * NC);
        const uint32_t f01 = f2 ? t[2] : t[0], f23 = f2 ? t[3] : t[1];
        const uint32_t F[4] = {f01 & 0xffffu, f01 >> 16, f23 & 0xffffu, f23 >> 16};
        const uint32_t s01 = s2 ? t[2] : t[0], s23 = s2 ? t[3] : t[1];
        const uint32_t S[4] = {s01 << 16, s01 & 0xffff0000u, s23 << 16, s23 & 0xffff0000u};
        uint32_t *dst = cftab + wv * (64 * SLOTS) + (32 * f2 + 16 * s2) * SLOTS + lane % SLOTS;
#pragma unroll
        for (int i = 0; i < 16; i++)
            dst[i * SLOTS] = F[((i >> 3) & 1) * 2 + ((i >> 1) & 1)] | S[((i >> 2) & 1) * 2 + (i & 1)];
    } else if constexpr (CF4) {
        // entry e = (f3 s3 f2 s2 f1 s1 f0 s0) holds (lut[f], lut[s]).  lane = (row, f3, s3), the group of waves is f2: a
        // lane writes the 32 entries (s2 f1 s1 f0 s0) of its eighth of the table from the halves of its row's values.
        const int f3 = lane >> 5, s3 = (lane >> 4) & 1;
        const u32x4 *row = reinterpret_cast<const u32x4 *>(lut + (size_t)min(n0 + (lane & 15), N - 1) * NC);
        const u32x4 lo = row[0], hi = row[1];  // values 0..7, 8..15
        const uint32_t fa = f3 ? (kh ? hi[2] : hi[0]) : (kh ? lo[2] : lo[0]);  // values 4 (2 f3 + f2) + {0, 1}
        const uint32_t fb = f3 ? (kh ? hi[3] : hi[1]) : (kh ? lo[3] : lo[1]);  // ... + {2, 3}
        const uint32_t F[4] = {fa & 0xffffu, fa >> 16, fb & 0xffffu, fb >> 16};
        uint32_t S[8];                                                           // values 8 s3 + 0..7, in the high half
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const uint32_t sv = s3 ? hi[k] : lo[k];
            S[2 * k] = sv << 16;
            S[2 * k + 1] = sv & 0xffff0000u;
        }
        uint32_t *dst = cftab + wv * (256 * 16) + ((f3 * 4 + s3 * 2 + kh) * 32) * 16 + (lane & 15);
#pragma unroll
        for (int i = 0; i < 32; i++)
            dst[i * 16] = F[((i >> 3) & 1) * 2 + ((i >> 1) & 1)] | S[((i >> 4) & 1) * 4 + ((i >> 2) & 1) * 2 + (i & 1)];
    } else if constexpr (CF16) {
        // lane = (row [, copy], part of the table); group kh copies its half of that part: 8 entries per 16-byte load,
        // a store covers 64 / SLOTS entries x SLOTS slots
        // (4 bits with one group: two parts of eight entries, written twice over)
        constexpr int PARTS = (kWave / SLOTS) * KH * 8 <= NC ? kWave / SLOTS : NC / 8 / KH, EPL = NC / PARTS / KH;
        static_assert(PARTS >= 1 && EPL % 8 == 0, "");
        const int e0 = ((lane / SLOTS) % PARTS) * (NC / PARTS) + kh * EPL;
        const u32x4 *src = reinterpret_cast<const u32x4 *>(lut + (size_t)min(n0 + (lane & 15), N - 1) * NC + e0);
        uint32_t *dst = cftab + wv * (NC * SLOTS) + e0 * SLOTS + (lane % SLOTS);
        u32x4 v[EPL / 8];
#pragma unroll
        for (int i = 0; i < EPL / 8; i++) v[i] = src[i];
#pragma unroll
        for (int i = 0; i < EPL / 8; i++)
#pragma unroll
            for (int d = 0; d < 4; d++) {
                dst[(8 * i + 2 * d) * SLOTS] = v[i][d] & 0xffffu;
                dst[(8 * i + 2 * d + 1) * SLOTS] = v[i][d] >> 16;
            }
    } else if constexpr (PAIR) {
        // each wave builds pair tables of its own rows (with two K halves: its half of them), eight rows' loads in
        // flight at a time
        const PairLane<BITS> pl = pair_lane<BITS>(lane);
#pragma unroll
        for (int r0 = 0; r0 < WROWS / KH; r0 += 8) {
            const int r1 = kh * (WROWS / KH) + r0;
            TableWords<BITS> tw[8];
#pragma unroll
            for (int i = 0; i < 8; i++) tw[i] = lookup_table_fetch<BITS>(lut + (size_t)min(n0 + r1 + i, N - 1) * NC, lane, pl);
#pragma unroll
            for (int i = 0; i < 8; i++) lookup_table_stage<BITS>(tw[i], &tables[wv * WROWS + r1 + i][0], lane);
        }
    } else {
        // the tables of the workgroup's rows are contiguous in lut (rows past N re-read the last 16 bytes of the array)
        constexpr int TQ = BN * NC / 8;  // 16-byte quads
        const u32x4 *src = reinterpret_cast<const u32x4 *>(lut);
        u32x4 *dst = reinterpret_cast<u32x4 *>(&tables[0][0]);
        const long long first = (long long)nb * (NC / 8), last = (long long)N * (NC / 8) - 1;
        for (int i = kh * NTHR + tid; i < TQ; i += KH * NTHR) dst[i] = src[min(first + i, last)];
    }
    __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0): the stages requested above are in LDS
    __syncthreads();

    typedef __attribute__((address_space(3))) uint16_t lds_u16_t;
    typedef __attribute__((address_space(3))) uint32_t lds_u32_t;
    // table reads are written as offsets from the tables array (not as bare LDS addresses), so that the compiler knows
    // they cannot touch a stage buffer a direct load is filling
    typedef __attribute__((address_space(3))) uint8_t lds_u8_t;
    const lds_u8_t *const tables_lds = (const lds_u8_t *)&tables[0][0];
    const uint32_t tab_base0 = (uint32_t)(wv * WROWS + col) * TB;  // byte offset of this lane's row table
    const lds_u8_t *const cftab_lds = (const lds_u8_t *)&cftab[0];
    const uint32_t cf_base = CF4 ? (uint32_t)(wv * (256 * 16) + (lane & 15)) * 4u
                                 : (uint32_t)(wv * ((CF16 ? NC : 64) * SLOTS) + lane % SLOTS) * 4u;  // ... of this lane's slot of entry 0

    float4_t acc[RB][MBW];
#pragma unroll
    for (int rb = 0; rb < RB; rb++)
#pragma unroll
        for (int mb = 0; mb < MBW; mb++) acc[rb][mb] = float4_t{0.f, 0.f, 0.f, 0.f};

    constexpr int PRE = BITS <= 7 ? 1 : 0;  // index bytes hold the byte offset into the table where that fits a byte
    constexpr int NRAW = PAIR ? 4 : 8;      // table reads per B operand
    uint32_t idx[4][RB][NRAW];              // indices of the 16 words of the step (lane: words 16 step + 4 wi + grp)
    half8_t afrag[2][MBW];                  // A operands of the octet in work and of the next one
    uint32_t braw[2][RB][NRAW];             // table entries of their B operands as they come from LDS
    // A operands of octet wi of the stage in buffer buf
    auto issue_a = [&](auto buf_c, auto wi_c, half8_t(&a)[MBW]) {
        constexpr int wi = decltype(wi_c)::value;
        auto &xt = stage_buffer(buf_c);
#pragma unroll
        for (int mb = 0; mb < MBW; mb++) a[mb] = __builtin_bit_cast(half8_t, xt[kh][mb * 16 + col][(4 * wi + grp) ^ col]);
    };
    // table reads for the eight weights of byte group j of word wi of each row block
    auto issue_b = [&](auto j_c, auto wi_c, uint32_t(&raw)[RB][NRAW]) {
        constexpr int c = 3 - decltype(j_c)::value, wi = decltype(wi_c)::value;
        static_for<RB>([&](auto rb_c) {
            constexpr int rb = decltype(rb_c)::value;
            const uint32_t tab_base = tab_base0 + rb * (kGemmRows * TB);
            static_for<NRAW>([&](auto e_c) {
                constexpr int i = decltype(e_c)::value;
                if constexpr (PAIR) {
                    // byte c of idx[i]: the entry of elements (2i, 2i+1) of byte group j -- at 3 bits already its byte offset
                    if constexpr (CF) {
                        // the index byte is 4 x entry
                        raw[rb][i] = *reinterpret_cast<const lds_u32_t *>(cftab_lds + (cf_base + byte_offset<c, ESHIFT - 2>(idx[wi][rb][i])));
                    } else if constexpr (CF4) {
                        // the index byte is the entry, of 64 bytes
                        raw[rb][i] = *reinterpret_cast<const lds_u32_t *>(cftab_lds + (cf_base + byte_offset<c, 6>(idx[wi][rb][i])));
                    } else {
                        uint32_t a0;
                        if constexpr (BITS == 3) a0 = byte_add<c>(tab_base, idx[wi][rb][i]);
                        else a0 = tab_base + byte_offset<c, 2>(idx[wi][rb][i]);
                        raw[rb][i] = *reinterpret_cast<const lds_u32_t *>(tables_lds + a0);
                    }
                } else {
                    if constexpr (CF16) {
                        // the index byte is 2 x entry; at 8 bits the entry
                        raw[rb][i] = *reinterpret_cast<const lds_u16_t *>(cftab_lds + (cf_base + byte_offset<c, ESHIFT - PRE>(idx[wi][rb][i])));
                    } else {
                        uint32_t a0;
                        if constexpr (PRE) a0 = byte_add<c>(tab_base, idx[wi][rb][i]);
                        else a0 = tab_base + byte_offset<c, 1>(idx[wi][rb][i]);
                        raw[rb][i] = *reinterpret_cast<const lds_u16_t *>(tables_lds + a0);
                    }
                }
            });
        });
    };
    // words past the row end: zero weights (their activations are zeros too)
    auto finish_b = [&](auto check_c, const uint32_t(&raw)[RB][NRAW], bool alive, half8_t(&b)[RB]) {
#pragma unroll
        for (int rb = 0; rb < RB; rb++) {
            u32x4 bw;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                uint32_t packed;
                if constexpr (PAIR) packed = raw[rb][i];
                else packed = raw[rb][2 * i] | (raw[rb][2 * i + 1] << 16);
                if constexpr (decltype(check_c)::value) bw[i] = alive ? packed : 0u;
                else bw[i] = packed;
            }
            b[rb] = __builtin_bit_cast(half8_t, bw);
        }
    };
    // One step.  CHECK: this step or the next (whose first stages are requested here) may reach past the end of the row
    // or of the walk; all other steps run without the selects that zero the weights of such words and that pick the
    // source of a unit.
    auto run_step = [&](auto check_c, int it) {
        constexpr bool CHECK = decltype(check_c)::value;
        const int step = step_at(it), step_next = step_at(it + 1);
        const bool active = active_at(it);
#pragma unroll
        for (int rb = 0; rb < RB; rb++) {
#pragma unroll
            for (int p = 0; p < BITS; p++) transpose_rows4(q[rb][p]);
#pragma unroll
            for (int wi = 0; wi < 4; wi++) {
                uint32_t qq[BITS];
#pragma unroll
                for (int p = 0; p < BITS; p++) qq[p] = q[rb][p][wi];
                if constexpr (PAIR) planes_to_adjacent_pairs<BITS>(qq, idx[wi][rb]);
                else planes_to_indices<BITS, PRE>(qq, idx[wi][rb]);
            }
        }
        const bool partial = 16 * (step + 1) > W;
        bool live[4];
#pragma unroll
        for (int wi = 0; wi < 4; wi++) live[wi] = !CHECK || (active && (!partial || 16 * step + 4 * wi + grp < W));

        // One stage = byte group j of the 16 words: four octets (wi), each RB B operands and MBW A operands feeding
        // RB x MBW matrix instructions.  The LDS reads of octet wi + 1 (A operands, table entries) are issued before
        // the matrix instructions of octet wi; scheduling fences pin that order.  The table reads of the first octet
        // of the next stage pass the barrier as well (the tables do not change).
        static_for<4>([&](auto j_c) {
            constexpr int j = decltype(j_c)::value, buf = j % NBUF;
            // the stage PD ahead goes into the buffer that the stage before this one was read from (every wave has
            // passed the barrier that ended it); past the end of the walk it fetches zeros that nobody reads
            stage_dma(check_c, it + ((j + PD) >> 2), (j + PD) & 3, std::integral_constant<int, (j + PD) % NBUF>{});
            if constexpr (j == 0) {
                // the planes of the next step are requested AFTER the direct loads of this stage: loads complete in
                // order, so the waits for stages below can leave the planes in flight.  (After the last step this
                // re-reads the planes of that step and uses nothing: the waits below count on these loads.)
                __builtin_amdgcn_sched_barrier(0);
                fetch(step_next, q);
                __builtin_amdgcn_sched_barrier(0);
            }
            issue_a(std::integral_constant<int, buf>{}, std::integral_constant<int, 0>{}, afrag[0]);
            if constexpr (j == 0) issue_b(j_c, std::integral_constant<int, 0>{}, braw[0]);
            static_for<4>([&](auto wi_c) {
                constexpr int wi = decltype(wi_c)::value, cur = wi & 1, nxt = cur ^ 1;
                half8_t bfrag[RB];
                finish_b(check_c, braw[cur], live[wi], bfrag);
                if constexpr (wi < 3) {
                    issue_a(std::integral_constant<int, buf>{}, std::integral_constant<int, wi + 1>{}, afrag[nxt]);
                    issue_b(j_c, std::integral_constant<int, wi + 1>{}, braw[nxt]);
                } else if constexpr (j < 3) {
                    issue_b(std::integral_constant<int, j + 1>{}, std::integral_constant<int, 0>{}, braw[nxt]);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int mb = 0; mb < MBW; mb++)
#pragma unroll
                    for (int rb = 0; rb < RB; rb++)
                        acc[rb][mb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(afrag[cur][mb], bfrag[rb], acc[rb][mb], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            });
            // The next stage must have landed; it was requested PD - 1 stages before this one.  Loads complete in order,
            // so what may stay outstanding is what was requested after it: the direct loads of the PD - 1 stages since
            // (MBW each) and, up to stage PD - 1 of a step, the plane loads of the next step.  Then this wave's LDS reads
            // of `buf` are done too (lgkmcnt(0)) and the workgroup meets.  The bare barrier instruction, not the fenced
            // form: the release fence makes the compiler wait for EVERY outstanding load here once direct loads are in
            // flight.
            constexpr int keep = (PD - 1) * MBW + (j <= PD - 1 ? BITS * RB : 0);
            static_assert(keep < 64, "");
            __builtin_amdgcn_s_waitcnt(0x0070 | (keep & 15) | ((keep >> 4) << 14));
            __builtin_amdgcn_s_barrier();
        });
    };
    // (tiles of 128 activation rows at 5..7 bits keep the one form with the selects: the second copy of the step costs
    // them the registers of their second wave per SIMD -- 11008 x 4096 at 256 rows, 5 bits: 91 us against 75; at 8 bits
    // the tables leave room for one workgroup per CU either way)
    for (int it = 0; it < nit; it++) {
        const int s0 = kh * nit + it;  // this step and the next, before clamping
        if ((MBW > 4 && BITS >= 5 && BITS <= 7) || s0 + 1 >= steps || 16 * (s0 + 2) > W)
            run_step(std::true_type{}, it);
        else
            run_step(std::false_type{}, it);
    }
    // the loads for stages past the end of the walk have landed too (they go where the partial tiles are parked below),
    // for every wave
    __builtin_amdgcn_s_waitcnt(0x0070);
    if constexpr (KH > 1) __syncthreads();

    // D[i][j]: lane l holds activation rows i = 4 (l / 16) + v of the block and weight row j = l % 16
    if constexpr (KH == 2) {
        // the last barrier of the loop has passed: nobody reads the stage buffers any more.  Group 1 parks its tiles in
        // its own buffers, group 0 adds them to its own.
        float *park = reinterpret_cast<float *>(&xt0[1][0][0]) + wv * (RB * MBW * 4 * kWave);
        if (kh == 1) {
#pragma unroll
            for (int rb = 0; rb < RB; rb++)
#pragma unroll
                for (int mb = 0; mb < MBW; mb++)
#pragma unroll
                    for (int v = 0; v < 4; v++) park[((rb * MBW + mb) * 4 + v) * kWave + lane] = acc[rb][mb][v];
        }
        __syncthreads();
        if (kh == 1) return;
#pragma unroll
        for (int rb = 0; rb < RB; rb++)
#pragma unroll
            for (int mb = 0; mb < MBW; mb++)
#pragma unroll
                for (int v = 0; v < 4; v++) acc[rb][mb][v] += park[((rb * MBW + mb) * 4 + v) * kWave + lane];
    }
#pragma unroll
    for (int rb = 0; rb < RB; rb++) {
        const int n = n0 + rb * kGemmRows + col;
#pragma unroll
        for (int mb = 0; mb < MBW; mb++)
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const int m = m0 + mb * 16 + 4 * grp + v;
                if (m < M && n < N) out[(size_t)m * ldo + n] = (half_t)acc[rb][mb][v];
            }
    }
}

}  // namespace ap

// Bitplane dequantiser for gfx950: out[n,k] = lut[n, index_b(n,k)], fp16 [N,K].
//
// Replaces the reference's dequant_kbit_store<bits>
// (any_precision/modules/kernels/dequant.cuh:177-242).  Result is a pure
// table copy, hence bit-exact by construction when the index is right.
//
// Mapping: the unit of work is one 64-word segment of one row (2048 elements); a wave
// takes segments in a grid-stride loop, lane l owns word l of the segment.  Per word a
// lane reads one dword per plane (a wave covers 256 B of each plane, fully coalesced),
// rebuilds its 32 indices in registers, gathers from the row's table in LDS and emits four
// 16-byte stores; for a fixed byte group the 32 lanes of a chunk write 512 contiguous
// bytes.  Cutting rows into segments keeps the number of independent waves proportional to
// the bytes, whatever the row length.  One launch serves up to kDequantMaxGroup linears (of any shapes, at one
// bit-width): their segments are numbered through and a wave finds the member of its segment with scalar selects.
#pragma once
#include "ap_bitplane.hpp"
#include "ap_device.hpp"
#include "ap_reciprocal.hpp"

namespace ap {

constexpr int kDequantWaves = 4;     // waves per workgroup
constexpr int kDequantMaxGroup = 8;  // linears one launch can serve (any shapes, one bit-width): a decoder layer has seven

// The linears of one launch, passed by value as kernel arguments.  The 64-word segments of all members are
// numbered through: member g owns items [item_end[g-1], item_end[g]); `items` is the total (below 2^31, the host
// checks).  seg_magic[g] = reciprocal_floor(S_g), S_g the segments of a row of member g (ap_reciprocal.hpp): the
// kernel divides an item number by S_g with one multiply and one correction step instead of a division.
struct DequantMembers {
    const uint32_t *qweight[kDequantMaxGroup];
    const uint16_t *lut[kDequantMaxGroup];
    uint16_t *out[kDequantMaxGroup];
    int N[kDequantMaxGroup];
    int K[kDequantMaxGroup];
    int item_end[kDequantMaxGroup];
    uint32_t seg_magic[kDequantMaxGroup];
    int items;
    int count;
};

// Where one item lives (all wave-uniform) and what its lane loads.
struct DequantItem {
    global_ptr<const char> planes;    // first plane word of the row
    global_ptr<const half_t> table;   // the row's table
    global_ptr<char> orow;            // the row's output
    size_t plane_bytes;
    int K, W, seg;
};

template <int BITS>
struct DequantLoads {
    LutRegs<BITS> table;
    uint32_t q[BITS];
};

// One wave walks its items; the loads of the item after the current one (its table row and its plane words) are
// issued before the current item's lookups and stores, so the memory round trip of an item is covered by the
// work of the one before it.  The two tables of a wave in LDS alternate with the items.  Within an item the order is: table fetch, plane loads, THEN the table goes to LDS
// (staging first would make the wave wait for its table before its plane loads leave).
template <int BITS>
__global__ __launch_bounds__(kDequantWaves * kWave) void dequant_kbit_kernel(const DequantMembers mem) {
    constexpr int NC = 1 << BITS;
    __shared__ __attribute__((aligned(16))) half_t tables[kDequantWaves][2][NC];

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);

    // Member 0 and the scalars of every item in ONE statement that wants them in scalar registers: one clause of
    // scalar loads, one wait (the compiler alone loads an argument where it is first used, a dependent round trip
    // each).  The fields of another member are read by index when an item belongs to it.
    const uint32_t *q0 = mem.qweight[0];
    const uint16_t *lut0 = mem.lut[0];
    uint16_t *out0 = mem.out[0];
    int N0 = mem.N[0], K0 = mem.K[0], count = mem.count, items = mem.items;
    uint32_t magic0 = mem.seg_magic[0];
    int e0 = mem.item_end[0], e1 = mem.item_end[1], e2 = mem.item_end[2], e3 = mem.item_end[3], e4 = mem.item_end[4],
        e5 = mem.item_end[5], e6 = mem.item_end[6];
    asm volatile("" : "+s"(q0), "+s"(lut0), "+s"(out0), "+s"(N0), "+s"(K0), "+s"(count), "+s"(items), "+s"(magic0),
                      "+s"(e0), "+s"(e1), "+s"(e2), "+s"(e3), "+s"(e4), "+s"(e5), "+s"(e6));

    auto locate = [&](int item) {
        const uint32_t *qw = q0;
        const uint16_t *lt = lut0;
        uint16_t *ot = out0;
        int N = N0, K = K0, first = 0;
        uint32_t magic = magic0;
        if (count > 1) {  // scalar branches: a plain call skips this
            // item_end ascends; the first term as integer arithmetic (1 when item >= e0: as a select of 1 and 0
            // it is compiled through a vector register)
            int g = (int)((uint32_t)(e0 - 1 - item) >> 31);
            g = (count > 2 && item >= e1) ? 2 : g;
            g = (count > 3 && item >= e2) ? 3 : g;
            g = (count > 4 && item >= e3) ? 4 : g;
            g = (count > 5 && item >= e4) ? 5 : g;
            g = (count > 6 && item >= e5) ? 6 : g;
            g = (count > 7 && item >= e6) ? 7 : g;
            if (g > 0) {
                qw = mem.qweight[g];
                lt = mem.lut[g];
                ot = mem.out[g];
                N = mem.N[g];
                K = mem.K[g];
                magic = mem.seg_magic[g];
                first = mem.item_end[g - 1];
            }
        }
        DequantItem it;
        it.K = K;
        it.W = K >> 5;
        const uint32_t S = (uint32_t)(it.W + kWave - 1) / kWave;  // segments per row
        const uint32_t local = (uint32_t)(item - first);
        uint32_t row, seg;
        divmod_by_reciprocal(local, S, magic, row, seg);
        it.seg = (int)seg;
        it.plane_bytes = (size_t)N * it.W * sizeof(uint32_t);
        it.planes = scalar_ptr(reinterpret_cast<const char *>(qw + (size_t)row * it.W));
        it.table = scalar_ptr(reinterpret_cast<const half_t *>(lt) + (size_t)row * NC);
        it.orow = scalar_ptr(reinterpret_cast<char *>(ot + (size_t)row * K));
        return it;
    };
    auto issue = [&](const DequantItem &it) {
        DequantLoads<BITS> r;
        r.table = lut_fetch<BITS>(it.table, lane);
        const uint32_t w = (uint32_t)(it.seg * kWave + lane);
        // lanes past the row end take word 0 of the segment (and later store what its own lane stores)
        const uint32_t byte = (w < (uint32_t)it.W ? w : (uint32_t)(it.seg * kWave)) * (uint32_t)sizeof(uint32_t);
#pragma unroll
        for (int p = 0; p < BITS; p++) r.q[p] = load_at_nt<uint32_t>(scalar_ptr(it.planes + p * it.plane_bytes), byte);
        return r;
    };
    auto finish = [&](const DequantItem &it, DequantLoads<BITS> &r, half_t *tab) {
        lut_arrive<BITS>(r.table);
        lut_stage<BITS>(r.table, tab, lane);
        // LDS operations of one wave complete in order, so the table is visible to the gathers below
        // without a workgroup barrier.
        __builtin_amdgcn_wave_barrier();
        // No branch on "is this lane's word inside the row": a lane past the row end has loaded word 0 of the
        // segment, computes what that word's own lane computes and stores the same bytes to the same addresses
        // (a duplicate within one store instruction).  So every load is consumed on every path, no store is a
        // "maybe", and each group of eight elements leaves as soon as its lookups are back.
        const int w = it.seg * kWave + lane;
        const int wv = w < it.W ? w : it.seg * kWave;
        uint32_t idx[8];
        planes_to_indices<BITS>(r.q, idx);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int sh = 8 * (3 - j);
            u32x4 v;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint16_t lo = __builtin_bit_cast(uint16_t, tab[(idx[2 * i] >> sh) & 0xffu]);
                const uint16_t hi = __builtin_bit_cast(uint16_t, tab[(idx[2 * i + 1] >> sh) & 0xffu]);
                v[i] = (uint32_t)lo | ((uint32_t)hi << 16);
            }
            store_at_nt(it.orow, (uint32_t)group_base(wv, j, it.K) * (uint32_t)sizeof(half_t), v);
        }
    };

    const int stride = (int)gridDim.x * kDequantWaves;
    int item = (int)blockIdx.x * kDequantWaves + wave;
    if (item >= items) return;
    // Two register sets take turns (the loop body is written out twice): one holds the item being finished, the
    // other receives the loads of the item after it.  Handing the prefetched registers over with copies instead
    // would make every iteration wait for those loads at its end.
    DequantItem item_a = locate(item), item_b;
    DequantLoads<BITS> loads_a = issue(item_a), loads_b;
    while (true) {
        if (item + stride >= items) {
            finish(item_a, loads_a, tables[wave][0]);
            break;
        }
        item += stride;
        item_b = locate(item);
        loads_b = issue(item_b);
        finish(item_a, loads_a, tables[wave][0]);
        if (item + stride >= items) {
            finish(item_b, loads_b, tables[wave][1]);
            break;
        }
        item += stride;
        item_a = locate(item);
        loads_a = issue(item_a);
        finish(item_b, loads_b, tables[wave][1]);
    }
}

}  // namespace ap

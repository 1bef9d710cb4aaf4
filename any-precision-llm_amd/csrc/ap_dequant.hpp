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

namespace ap {

constexpr int kDequantWaves = 4;     // waves per workgroup
constexpr int kDequantMaxGroup = 8;  // linears one launch can serve (any shapes, one bit-width): a decoder layer has seven

// The linears of one launch, passed by value as kernel arguments.  The 64-word segments of all members are
// numbered through: member g owns items [item_end[g-1], item_end[g]).
struct DequantMembers {
    const uint32_t *qweight[kDequantMaxGroup];
    const uint16_t *lut[kDequantMaxGroup];
    uint16_t *out[kDequantMaxGroup];
    int N[kDequantMaxGroup];
    int K[kDequantMaxGroup];
    long long item_end[kDequantMaxGroup];
    int count;
};

template <int BITS>
__global__ __launch_bounds__(kDequantWaves * kWave) void dequant_kbit_kernel(const DequantMembers mem) {
    constexpr int NC = 1 << BITS;
    __shared__ __attribute__((aligned(16))) half_t tables[kDequantWaves][2][NC];

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const long long items = mem.item_end[mem.count - 1];
    const long long stride = (long long)gridDim.x * kDequantWaves;

    int buf = 0;
    for (long long item = (long long)blockIdx.x * kDequantWaves + wave; item < items; item += stride, buf ^= 1) {
        // the member this item belongs to (scalar selects; no indexed access to the arguments)
        const uint32_t *__restrict__ qweight = mem.qweight[0];
        const half_t *__restrict__ lut = reinterpret_cast<const half_t *>(mem.lut[0]);
        half_t *__restrict__ out = reinterpret_cast<half_t *>(mem.out[0]);
        int N = mem.N[0], K = mem.K[0];
        long long first = 0;
#pragma unroll
        for (int g = 1; g < kDequantMaxGroup; g++) {
            if (g < mem.count && item >= mem.item_end[g - 1]) {
                qweight = mem.qweight[g];
                lut = reinterpret_cast<const half_t *>(mem.lut[g]);
                out = reinterpret_cast<half_t *>(mem.out[g]);
                N = mem.N[g];
                K = mem.K[g];
                first = mem.item_end[g - 1];
            }
        }
        const int W = K >> 5;
        const int S = (W + kWave - 1) / kWave;  // segments per row
        const size_t plane_stride = (size_t)N * W;
        const uint32_t local = (uint32_t)(item - first);  // a member has fewer than 2^31 segments (checked by the host)
        const int row = (int)(local / (uint32_t)S), seg = (int)(local - (uint32_t)row * (uint32_t)S);
        half_t *tab = tables[wave][buf];
        lut_stage<BITS>(lut_fetch<BITS>(lut + (size_t)row * NC, lane), tab, lane);
        // LDS operations of one wave complete in order, so the table is
        // visible to the gathers below without a workgroup barrier.
        __builtin_amdgcn_wave_barrier();

        const int w = seg * kWave + lane;
        if (w < W) {
            const uint32_t *wrow = qweight + (size_t)row * W;
            half_t *orow = out + (size_t)row * K;
            uint32_t q[BITS];
#pragma unroll
            for (int p = 0; p < BITS; p++) q[p] = __builtin_nontemporal_load(wrow + p * plane_stride + w);
            uint32_t idx[8];
            planes_to_indices<BITS>(q, idx);
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
                __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(orow + group_base(w, j, K)));
            }
        }
    }
}

}  // namespace ap

// Measurement aid: a kernel that only reads memory, as fast as this library knows how to, so that a
// benchmark can put "what the machine does for these bytes" beside a GEMV over the same buffers.
#pragma once
#include "ap_device.hpp"

namespace ap {

constexpr int kProbeWaves = 4;  // waves per workgroup

// Reads `units0` + `units1` 16-byte units (two buffers: the planes and the tables of a linear) with
// non-temporal 16-byte loads, four in flight per lane, xors them together and stores one dword per
// lane that saw anything nonzero-or-not (the store keeps the loads alive; its value is meaningless).
__global__ __launch_bounds__(kProbeWaves *kWave) void probe_stream_kernel(const u32x4 *__restrict__ buf0, long long units0,
                                                                           const u32x4 *__restrict__ buf1, long long units1,
                                                                           uint32_t *__restrict__ sink) {
    const long long tid = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const long long stride = (long long)gridDim.x * blockDim.x;
    u32x4 acc = {0u, 0u, 0u, 0u};
    auto sweep = [&](const u32x4 *__restrict__ buf, long long units) {
        long long i = tid;
        for (; i + 3 * stride < units; i += 4 * stride) {
            const u32x4 a = __builtin_nontemporal_load(buf + i);
            const u32x4 b = __builtin_nontemporal_load(buf + i + stride);
            const u32x4 c = __builtin_nontemporal_load(buf + i + 2 * stride);
            const u32x4 d = __builtin_nontemporal_load(buf + i + 3 * stride);
            acc ^= a ^ b ^ c ^ d;
        }
        for (; i < units; i += stride) acc ^= __builtin_nontemporal_load(buf + i);
    };
    sweep(buf0, units0);
    sweep(buf1, units1);
    const uint32_t v = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
    if (v == 0x9e3779b9u) sink[0] = v;  // practically never true: no store traffic, loads stay live
}

// Only WRITES `units` 16-byte units (non-temporal stores of a constant): what the machine does for the
// output of a kernel that is bound by its stores, such as the dequantiser.
__global__ __launch_bounds__(kProbeWaves *kWave) void probe_write_kernel(u32x4 *__restrict__ dst, long long units,
                                                                          uint32_t value) {
    const long long tid = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const long long stride = (long long)gridDim.x * blockDim.x;
    const u32x4 v = {value, value, value, value};
    for (long long i = tid; i < units; i += stride) __builtin_nontemporal_store(v, dst + i);
}

// A kernel that does nothing: the fixed cost of a launch.
__global__ void probe_empty_kernel(uint32_t *sink) {
    if (threadIdx.x == 0x7fffffffu) sink[0] = 0u;  // never true: the kernel keeps its argument and stores nothing
}

}  // namespace ap

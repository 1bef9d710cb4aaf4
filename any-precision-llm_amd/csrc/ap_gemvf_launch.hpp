// Host-side launch interface of the fine-grained GEMV kernels (ap_gemvf.hpp); one translation
// unit per bit-width (ap_gemvf_inst.hip with -DAP_BITS=b).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ap {

constexpr int kGemvfMaxSeg = 16;  // K-segments (waves) per workgroup: rows of up to 32768 elements
constexpr int kGemvfMaxM = 4;     // activation rows

struct GemvfGeometry {
    int S;     // K-segments of 2048 elements = waves per workgroup
    int grid;  // workgroups = row pairs
};

// Launches gemvf_kbit_kernel<BITS, M, *> on `stream`.  1 <= M <= kGemvfMaxM, N even, K a multiple of 64.
template <int BITS>
void launch_gemvf(int M, const GemvfGeometry &geo, const uint16_t *x, const uint32_t *qweight, const uint16_t *lut,
                  uint16_t *out, int N, int K, hipStream_t stream);

extern template void launch_gemvf<3>(int, const GemvfGeometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, hipStream_t);
extern template void launch_gemvf<4>(int, const GemvfGeometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, hipStream_t);
extern template void launch_gemvf<5>(int, const GemvfGeometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, hipStream_t);
extern template void launch_gemvf<6>(int, const GemvfGeometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, hipStream_t);
extern template void launch_gemvf<7>(int, const GemvfGeometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, hipStream_t);
extern template void launch_gemvf<8>(int, const GemvfGeometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, hipStream_t);

}  // namespace ap

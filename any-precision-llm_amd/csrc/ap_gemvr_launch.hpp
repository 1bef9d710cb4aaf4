// Host-side launch interface of the persistent GEMV kernels (ap_gemvr.hpp); one translation
// unit per bit-width (ap_gemvr_inst.hip with -DAP_BITS=b).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ap {

constexpr int kGemvrMaxSeg = 16;  // K-segments (waves) per workgroup: rows of up to 65536 elements
constexpr int kGemvrMaxM = 4;     // activation rows

struct GemvrGeometry {
    int S;     // K-segments of 4096 elements = waves per workgroup
    int grid;  // workgroups; workgroup g walks the rows g, g + grid, ...
};

// Launches gemvr_kbit_kernel<BITS, M, *> on `stream`.  1 <= M <= kGemvrMaxM, K a multiple of 64.
template <int BITS>
void launch_gemvr(int M, const GemvrGeometry &geo, const uint16_t *x, const uint32_t *qweight, const uint16_t *lut,
                  uint16_t *out, int N, int K, hipStream_t stream);

extern template void launch_gemvr<3>(int, const GemvrGeometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, hipStream_t);
extern template void launch_gemvr<4>(int, const GemvrGeometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, hipStream_t);
extern template void launch_gemvr<5>(int, const GemvrGeometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, hipStream_t);
extern template void launch_gemvr<6>(int, const GemvrGeometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, hipStream_t);
extern template void launch_gemvr<7>(int, const GemvrGeometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, hipStream_t);
extern template void launch_gemvr<8>(int, const GemvrGeometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, hipStream_t);

}  // namespace ap

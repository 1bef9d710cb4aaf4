// Host-side launch interface of the row-streaming GEMV kernels (ap_gemvp.hpp); one translation
// unit per bit-width (ap_gemvp_inst.hip with -DAP_BITS=b).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ap {

constexpr int kGemvpMaxSeg = 16;  // K-segments (waves) per workgroup: rows of up to 65536 elements
constexpr int kGemvpMaxM = 4;     // activation rows

struct GemvpGeometry {
    int S;     // K-segments of 4096 elements = waves per workgroup
    int grid;  // workgroups; workgroup g walks the row pairs g, g + grid, ...
};

// Launches gemvp_kbit_kernel<BITS, M, *> on `stream`.  1 <= M <= kGemvpMaxM, N even, K a multiple of 128.
template <int BITS>
void launch_gemvp(int M, const GemvpGeometry &geo, const uint16_t *x, const uint32_t *qweight, const uint16_t *lut,
                  uint16_t *out, int N, int K, hipStream_t stream);

extern template void launch_gemvp<3>(int, const GemvpGeometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, hipStream_t);
extern template void launch_gemvp<4>(int, const GemvpGeometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, hipStream_t);
extern template void launch_gemvp<5>(int, const GemvpGeometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, hipStream_t);
extern template void launch_gemvp<6>(int, const GemvpGeometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, hipStream_t);
extern template void launch_gemvp<7>(int, const GemvpGeometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, hipStream_t);
extern template void launch_gemvp<8>(int, const GemvpGeometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, hipStream_t);

}  // namespace ap

// Host-side launch interface of the tiled fused GEMM kernels (one translation unit per bit-width:
// ap_gemmt_inst.hip with -DAP_BITS=b).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ap {

constexpr int kGemmtWaves = 4;  // waves per workgroup, each on its own block(s) of 16 weight rows

struct GemmtGeometry {
    int mbw;     // blocks of 16 activation rows per workgroup tile (4 or 8); a workgroup owns 64 weight rows
    int kh;      // groups of four waves per workgroup, each on its share of K (1, or 2 with mbw = 4)
    int grid_n;  // ceil(N / 64)
    int grid_m;  // ceil(M / (16 mbw))
};

// Launches gemmt_kbit_kernel<BITS, 1, geo.mbw, geo.kh> on `stream`.  K must be a multiple of 128.
template <int BITS>
void launch_gemmt(const GemmtGeometry &geo, const uint16_t *x, const uint32_t *qweight, const uint16_t *lut,
                  uint16_t *out, int M, int N, int K, hipStream_t stream);

extern template void launch_gemmt<3>(const GemmtGeometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, int, hipStream_t);
extern template void launch_gemmt<4>(const GemmtGeometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, int, hipStream_t);
extern template void launch_gemmt<5>(const GemmtGeometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, int, hipStream_t);
extern template void launch_gemmt<6>(const GemmtGeometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, int, hipStream_t);
extern template void launch_gemmt<7>(const GemmtGeometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, int, hipStream_t);
extern template void launch_gemmt<8>(const GemmtGeometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, int, hipStream_t);

}  // namespace ap

// Host-side launch interface of the row-walking fused GEMM kernels (one translation unit per
// bit-width: ap_gemmw_inst.hip with -DAP_BITS=b).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ap {

constexpr int kGemmwMaxM = 32;  // activation rows (two MFMA row blocks with one step per wave)

struct GemmwGeometry {
    int mb;    // activation row blocks of 16 (1 or 2)
    int spw;   // steps of 512 elements per wave (1 or 2); mb * spw <= 2
    int ks;    // K-split waves per workgroup = ceil(steps / spw), 4..8
    int grid;  // workgroups, each walking blocks of 16 weight rows g, g + grid, ...
};

// Launches gemmw_kbit_kernel<BITS, geo.mb, geo.spw> on `stream`.
template <int BITS>
void launch_gemmw(const GemmwGeometry &geo, const uint16_t *x, const uint32_t *qweight, const uint16_t *lut,
                  uint16_t *out, int M, int N, int K, hipStream_t stream);

extern template void launch_gemmw<3>(const GemmwGeometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, int, hipStream_t);
extern template void launch_gemmw<4>(const GemmwGeometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, int, hipStream_t);
extern template void launch_gemmw<5>(const GemmwGeometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, int, hipStream_t);
extern template void launch_gemmw<6>(const GemmwGeometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, int, hipStream_t);
extern template void launch_gemmw<7>(const GemmwGeometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, int, hipStream_t);
extern template void launch_gemmw<8>(const GemmwGeometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, int, hipStream_t);

}  // namespace ap

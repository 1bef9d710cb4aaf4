// Persistent GEMV kernels of one bit-width (compile with -DAP_BITS=3..8) and their launch dispatch.
#include "ap_gemvr.hpp"

#ifndef AP_BITS
#error "compile with -DAP_BITS=<3..8>"
#endif

namespace ap {
namespace {

template <int BITS, int M>
void launch_m(const GemvrGeometry &geo, const half_t *x, const uint32_t *qweight, const half_t *lut, half_t *out, int N,
              int K, hipStream_t stream) {
    const dim3 block(kWave, geo.S), grid(geo.grid);
    // smallest workgroup bound that holds S waves: leaves the most registers per lane
    if (geo.S == 1)
        gemvr_kbit_kernel<BITS, M, 64><<<grid, block, 0, stream>>>(x, qweight, lut, out, N, K);
    else if (geo.S <= 4)
        gemvr_kbit_kernel<BITS, M, 256><<<grid, block, 0, stream>>>(x, qweight, lut, out, N, K);
    else if (geo.S <= 8)
        gemvr_kbit_kernel<BITS, M, 512><<<grid, block, 0, stream>>>(x, qweight, lut, out, N, K);
    else
        gemvr_kbit_kernel<BITS, M, 1024><<<grid, block, 0, stream>>>(x, qweight, lut, out, N, K);
}

}  // namespace

template <int BITS>
void launch_gemvr(int M, const GemvrGeometry &geo, const uint16_t *x, const uint32_t *qweight, const uint16_t *lut,
                  uint16_t *out, int N, int K, hipStream_t stream) {
    const half_t *xh = reinterpret_cast<const half_t *>(x);
    const half_t *lh = reinterpret_cast<const half_t *>(lut);
    half_t *oh = reinterpret_cast<half_t *>(out);
    switch (M) {
        case 1: return launch_m<BITS, 1>(geo, xh, qweight, lh, oh, N, K, stream);
        case 2: return launch_m<BITS, 2>(geo, xh, qweight, lh, oh, N, K, stream);
        case 3: return launch_m<BITS, 3>(geo, xh, qweight, lh, oh, N, K, stream);
        default: return launch_m<BITS, 4>(geo, xh, qweight, lh, oh, N, K, stream);
    }
}

template void launch_gemvr<AP_BITS>(int, const GemvrGeometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, hipStream_t);

}  // namespace ap

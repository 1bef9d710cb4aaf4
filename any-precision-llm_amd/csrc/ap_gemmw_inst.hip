// Row-walking fused GEMM kernels of one bit-width (compile with -DAP_BITS=3..8) and their launch dispatch.
#include "ap_gemmw.hpp"
#include "ap_gemmw_launch.hpp"

#ifndef AP_BITS
#error "compile with -DAP_BITS=<3..8>"
#endif

namespace ap {

template <int BITS>
void launch_gemmw(const GemmwGeometry &geo, const uint16_t *x, const uint32_t *qweight, const uint16_t *lut,
                  uint16_t *out, int M, int N, int K, hipStream_t stream) {
    const half_t *xh = reinterpret_cast<const half_t *>(x), *lh = reinterpret_cast<const half_t *>(lut);
    half_t *oh = reinterpret_cast<half_t *>(out);
    const dim3 block(kWave, geo.ks), grid(geo.grid);
    if (geo.mb == 2)
        gemmw_kbit_kernel<BITS, 2, 1><<<grid, block, 0, stream>>>(xh, qweight, lh, oh, M, N, K);
    else if (geo.spw == 2)
        gemmw_kbit_kernel<BITS, 1, 2><<<grid, block, 0, stream>>>(xh, qweight, lh, oh, M, N, K);
    else
        gemmw_kbit_kernel<BITS, 1, 1><<<grid, block, 0, stream>>>(xh, qweight, lh, oh, M, N, K);
}

template void launch_gemmw<AP_BITS>(const GemmwGeometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *,
                                    int, int, int, hipStream_t);

}  // namespace ap

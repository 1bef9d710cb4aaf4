// Fused GEMM kernels of one bit-width (compile with -DAP_BITS=3..8) and their launch dispatch.
#include "ap_gemm.hpp"
#include "ap_gemm_launch.hpp"

#ifndef AP_BITS
#error "compile with -DAP_BITS=<3..8>"
#endif

namespace ap {

template <int BITS>
void launch_gemm(const GemmGeometry &geo, const uint16_t *x, const uint32_t *qweight, const uint16_t *lut,
                 uint16_t *out, int M, int N, int K, hipStream_t stream) {
    const half_t *xh = reinterpret_cast<const half_t *>(x), *lh = reinterpret_cast<const half_t *>(lut);
    half_t *oh = reinterpret_cast<half_t *>(out);
    const dim3 block(kWave, geo.ks), grid(geo.grid);
    switch (geo.mb) {
        case 1: gemm_kbit_kernel<BITS, 1><<<grid, block, 0, stream>>>(xh, qweight, lh, oh, M, N, K); break;
        case 2: gemm_kbit_kernel<BITS, 2><<<grid, block, 0, stream>>>(xh, qweight, lh, oh, M, N, K); break;
        case 3: gemm_kbit_kernel<BITS, 3><<<grid, block, 0, stream>>>(xh, qweight, lh, oh, M, N, K); break;
        case 4: gemm_kbit_kernel<BITS, 4><<<grid, block, 0, stream>>>(xh, qweight, lh, oh, M, N, K); break;
        case 5: gemm_kbit_kernel<BITS, 5><<<grid, block, 0, stream>>>(xh, qweight, lh, oh, M, N, K); break;
        case 6: gemm_kbit_kernel<BITS, 6><<<grid, block, 0, stream>>>(xh, qweight, lh, oh, M, N, K); break;
        case 7: gemm_kbit_kernel<BITS, 7><<<grid, block, 0, stream>>>(xh, qweight, lh, oh, M, N, K); break;
        default: gemm_kbit_kernel<BITS, 8><<<grid, block, 0, stream>>>(xh, qweight, lh, oh, M, N, K); break;
    }
}

template void launch_gemm<AP_BITS>(const GemmGeometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *,
                                   int, int, int, hipStream_t);

}  // namespace ap

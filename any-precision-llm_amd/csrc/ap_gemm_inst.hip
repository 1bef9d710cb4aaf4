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
    const bool vec4 = ((K >> 5) & 3) == 0;  // whole 16-byte quads of words per row
    const uint32_t ks_magic = reciprocal_ceil((uint32_t)geo.ks);  // the kernel divides its step counts by ks with one multiplication
#define AP_GEMM_LAUNCH(MBV, MPV)                                                                                     \
    do {                                                                                                             \
        if (vec4) gemm_kbit_kernel<BITS, MBV, true, MPV, 1><<<grid, block, 0, stream>>>(xh, qweight, lh, oh, M, N, K, geo.ks, ks_magic);   \
        else gemm_kbit_kernel<BITS, MBV, false, MPV, 1><<<grid, block, 0, stream>>>(xh, qweight, lh, oh, M, N, K, geo.ks, ks_magic);       \
    } while (0)
#define AP_GEMM_CASE(MBV) \
    case MBV: AP_GEMM_LAUNCH(MBV, 0); break;
    if (geo.rb == 2) {  // chosen by the caller only with vec4 and at most two activation row blocks
        if (geo.mb == 1) gemm_kbit_kernel<BITS, 1, true, 0, 2><<<grid, block, 0, stream>>>(xh, qweight, lh, oh, M, N, K, geo.ks, ks_magic);
        else gemm_kbit_kernel<BITS, 2, true, 32, 2><<<grid, block, 0, stream>>>(xh, qweight, lh, oh, M, N, K, geo.ks, ks_magic);
        return;
    }
    if (geo.lookahead && vec4 && geo.mb <= 2) {
        if (geo.mb == 1) gemm_kbit_kernel<BITS, 1, true, 0, 1, true><<<grid, block, 0, stream>>>(xh, qweight, lh, oh, M, N, K, geo.ks, ks_magic);
        else gemm_kbit_kernel<BITS, 2, true, 32, 1, true><<<grid, block, 0, stream>>>(xh, qweight, lh, oh, M, N, K, geo.ks, ks_magic);
        return;
    }
    switch (geo.mb) {
        AP_GEMM_CASE(1)
        case 2: AP_GEMM_LAUNCH(2, 32); break;
        AP_GEMM_CASE(3) AP_GEMM_CASE(4) AP_GEMM_CASE(5) AP_GEMM_CASE(6) AP_GEMM_CASE(7)
        default: AP_GEMM_LAUNCH(8, 0); break;
    }
#undef AP_GEMM_LAUNCH
#undef AP_GEMM_CASE
}

template void launch_gemm<AP_BITS>(const GemmGeometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *,
                                   int, int, int, hipStream_t);

}  // namespace ap

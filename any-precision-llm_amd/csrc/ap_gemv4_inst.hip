// 4x4x4 matrix-core skinny GEMM kernels of one bit-width (compile with -DAP_BITS=3..8) and
// their launch dispatch.
#include "ap_gemv4.hpp"

#ifndef AP_BITS
#error "compile with -DAP_BITS=<3..8>"
#endif

namespace ap {
namespace {

template <int BITS, int MG, int G, int RQ>
void launch_rq(const Gemv4Geometry &geo, const half_t *x, const uint32_t *qweight, const half_t *lut, half_t *out,
              int M, int N, int K, hipStream_t stream) {
    const dim3 block(kWave, geo.S), grid(geo.grid);
    // smallest workgroup bound that holds S waves
    if (geo.S <= 4)
        gemv4_kbit_kernel<BITS, MG, G, RQ, 256><<<grid, block, 0, stream>>>(x, qweight, lut, out, M, N, K, geo.S);
    else if (geo.S <= 8)
        gemv4_kbit_kernel<BITS, MG, G, RQ, 512><<<grid, block, 0, stream>>>(x, qweight, lut, out, M, N, K, geo.S);
    else
        gemv4_kbit_kernel<BITS, MG, G, RQ, 1024><<<grid, block, 0, stream>>>(x, qweight, lut, out, M, N, K, geo.S);
}

template <int BITS>
void launch_one_group(const Gemv4Geometry &geo, const half_t *x, const uint32_t *qweight, const half_t *lut, half_t *out,
                      int M, int N, int K, hipStream_t stream) {
    switch (geo.G) {  // up to 4 activation rows: two row quads per workgroup measured best
        case 1: return launch_rq<BITS, 1, 1, 2>(geo, x, qweight, lut, out, M, N, K, stream);
        case 2: return launch_rq<BITS, 1, 2, 2>(geo, x, qweight, lut, out, M, N, K, stream);
        default: return launch_rq<BITS, 1, 4, 2>(geo, x, qweight, lut, out, M, N, K, stream);
    }
}

// 5..8 activation rows: four row quads per workgroup (the activations, twice as many, are then read
// half as often), one word group per wave, at most 8 waves
template <int BITS>
void launch_two_groups(const Gemv4Geometry &geo, const half_t *x, const uint32_t *qweight, const half_t *lut,
                       half_t *out, int M, int N, int K, hipStream_t stream) {
    const dim3 block(kWave, geo.S), grid(geo.grid);
    if (geo.S <= 4)
        gemv4_kbit_kernel<BITS, 2, 1, 4, 256><<<grid, block, 0, stream>>>(x, qweight, lut, out, M, N, K, geo.S);
    else
        gemv4_kbit_kernel<BITS, 2, 1, 4, 512><<<grid, block, 0, stream>>>(x, qweight, lut, out, M, N, K, geo.S);
}

}  // namespace

template <int BITS>
void launch_gemv4(const Gemv4Geometry &geo, const uint16_t *x, const uint32_t *qweight, const uint16_t *lut,
                  uint16_t *out, int M, int N, int K, hipStream_t stream) {
    const half_t *xh = reinterpret_cast<const half_t *>(x), *lh = reinterpret_cast<const half_t *>(lut);
    half_t *oh = reinterpret_cast<half_t *>(out);
    if (geo.mg == 1) return launch_one_group<BITS>(geo, xh, qweight, lh, oh, M, N, K, stream);
    launch_two_groups<BITS>(geo, xh, qweight, lh, oh, M, N, K, stream);
}

template void launch_gemv4<AP_BITS>(const Gemv4Geometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *,
                                    int, int, int, hipStream_t);

}  // namespace ap

// GEMV kernels of one bit-width (compile with -DAP_BITS=3..8) and their launch dispatch.
#include "ap_gemv.hpp"
#include "ap_gemv_launch.hpp"

#ifndef AP_BITS
#error "compile with -DAP_BITS=<3..8>"
#endif

namespace ap {
namespace {

template <int BITS, int M, int WPL, int R>
void launch_rows(const GemvGeometry &geo, const half_t *x, const GemvMembers &mem, int K, hipStream_t stream) {
    const dim3 block(kWave, geo.S), grid(geo.grid);
    // smallest workgroup bound that holds S waves: leaves the most registers per lane
    if (geo.S <= 4)
        gemv_kbit_kernel<BITS, M, WPL, R, 256><<<grid, block, 0, stream>>>(x, mem, K, geo.S);
    else if (geo.S <= 8)
        gemv_kbit_kernel<BITS, M, WPL, R, 512><<<grid, block, 0, stream>>>(x, mem, K, geo.S);
    else
        gemv_kbit_kernel<BITS, M, WPL, R, 1024><<<grid, block, 0, stream>>>(x, mem, K, geo.S);
}

template <int BITS, int M>
void launch_m(const GemvGeometry &geo, const half_t *x, const GemvMembers &mem, int K, hipStream_t stream) {
    if constexpr (M <= 2) {  // two words per lane and one row per workgroup exist for M <= 2 only
        if (geo.wpl == 2) {
            if (geo.R == 2) return launch_rows<BITS, M, 2, 2>(geo, x, mem, K, stream);
            return launch_rows<BITS, M, 2, 1>(geo, x, mem, K, stream);
        }
        if (geo.R == 1) return launch_rows<BITS, M, 1, 1>(geo, x, mem, K, stream);
    }
    if constexpr (M <= 4) {  // four rows per workgroup exist for up to four activation rows
        if (geo.R == 4) return launch_rows<BITS, M, 1, 4>(geo, x, mem, K, stream);
    }
    launch_rows<BITS, M, 1, 2>(geo, x, mem, K, stream);
}

template <int BITS, int M>
void launch_pair_m(const GemvGeometry &geo, const half_t *x, const GemvMembers &mem, int K, hipStream_t stream) {
    const dim3 block(kWave, geo.S), grid(geo.grid);
    if (geo.S <= 4)
        gemv_kbit_kernel<BITS, M, 1, 2, 256, true><<<grid, block, 0, stream>>>(x, mem, K, geo.S);
    else if (geo.S <= 8)
        gemv_kbit_kernel<BITS, M, 1, 2, 512, true><<<grid, block, 0, stream>>>(x, mem, K, geo.S);
    else
        gemv_kbit_kernel<BITS, M, 1, 2, 1024, true><<<grid, block, 0, stream>>>(x, mem, K, geo.S);
}

}  // namespace

template <int BITS>
void launch_gemv_pair(int M, const GemvGeometry &geo, const uint16_t *x, const GemvMembers &mem, int K, hipStream_t stream) {
    const half_t *xh = reinterpret_cast<const half_t *>(x);
    switch (M) {
        case 1: return launch_pair_m<BITS, 1>(geo, xh, mem, K, stream);
        case 2: return launch_pair_m<BITS, 2>(geo, xh, mem, K, stream);
        case 3: return launch_pair_m<BITS, 3>(geo, xh, mem, K, stream);
        default: return launch_pair_m<BITS, 4>(geo, xh, mem, K, stream);
    }
}

template void launch_gemv_pair<AP_BITS>(int, const GemvGeometry &, const uint16_t *, const GemvMembers &, int, hipStream_t);

template <int BITS>
void launch_gemv(int M, const GemvGeometry &geo, const uint16_t *x, const GemvMembers &mem, int K, hipStream_t stream) {
    const half_t *xh = reinterpret_cast<const half_t *>(x);
    switch (M) {
        case 1: return launch_m<BITS, 1>(geo, xh, mem, K, stream);
        case 2: return launch_m<BITS, 2>(geo, xh, mem, K, stream);
        case 3: return launch_m<BITS, 3>(geo, xh, mem, K, stream);
        case 4: return launch_m<BITS, 4>(geo, xh, mem, K, stream);
        case 5: return launch_m<BITS, 5>(geo, xh, mem, K, stream);
        case 6: return launch_m<BITS, 6>(geo, xh, mem, K, stream);
        case 7: return launch_m<BITS, 7>(geo, xh, mem, K, stream);
        default: return launch_m<BITS, 8>(geo, xh, mem, K, stream);
    }
}

template void launch_gemv<AP_BITS>(int, const GemvGeometry &, const uint16_t *, const GemvMembers &, int, hipStream_t);

}  // namespace ap

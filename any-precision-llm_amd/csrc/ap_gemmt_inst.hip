// Tiled fused GEMM kernels of one bit-width (compile with -DAP_BITS=3..8) and their launch dispatch.
#include "ap_gemmt.hpp"
#include "ap_gemmt_launch.hpp"

#ifndef AP_BITS
#error "compile with -DAP_BITS=<3..8>"
#endif

namespace ap {

template <int BITS>
void launch_gemmt(const GemmtGeometry &geo, const uint16_t *x, const GemmtMembers &members, int M, int K, hipStream_t stream) {
    const half_t *xh = reinterpret_cast<const half_t *>(x);
    // one-dimensional grid, weight-row tiles padded to groups of 8 (the kernel maps a workgroup to its tile)
    const dim3 block(kWave, kGemmtWaves * geo.kh), grid((unsigned)((geo.grid_n + 7) / 8 * 8) * (unsigned)geo.grid_m);
    // the kernel divides its workgroup number by tile_div with one multiplication (ap_reciprocal.hpp; grids stay below 2^31)
    const uint32_t tiles_pad = (uint32_t)((geo.grid_n + 7) / 8 * 8);
    const uint32_t tile_div = geo.grid_m <= 8 ? 8u * (uint32_t)geo.grid_m : tiles_pad, tile_magic = reciprocal_floor(tile_div);
    // one block of 16 weight rows per wave: two measured slower on every shape (a quarter of the workgroups, and the
    // LDS traffic per matrix instruction falls by less than a third)
    if (geo.mbw == 8)
        gemmt_kbit_kernel<BITS, 1, 8, 1><<<grid, block, 0, stream>>>(xh, members, M, K, geo.grid_m, tile_div, tile_magic);
    else if (geo.mbw == 1)
        gemmt_kbit_kernel<BITS, 1, 1, 2><<<grid, block, 0, stream>>>(xh, members, M, K, geo.grid_m, tile_div, tile_magic);
    else if (geo.mbw == 2)
        gemmt_kbit_kernel<BITS, 1, 2, 2><<<grid, block, 0, stream>>>(xh, members, M, K, geo.grid_m, tile_div, tile_magic);
    else if (geo.kh == 2)
        gemmt_kbit_kernel<BITS, 1, 4, 2><<<grid, block, 0, stream>>>(xh, members, M, K, geo.grid_m, tile_div, tile_magic);
    else
        gemmt_kbit_kernel<BITS, 1, 4, 1><<<grid, block, 0, stream>>>(xh, members, M, K, geo.grid_m, tile_div, tile_magic);
}

template void launch_gemmt<AP_BITS>(const GemmtGeometry &, const uint16_t *, const GemmtMembers &, int, int, hipStream_t);

}  // namespace ap

// Host-side launch interface of the tiled fused GEMM kernels (one translation unit per bit-width:
// ap_gemmt_inst.hip with -DAP_BITS=b).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ap {

constexpr int kGemmtWaves = 4;  // waves per workgroup, each on its own block(s) of 16 weight rows

struct GemmtGeometry {
    int mbw;     // blocks of 16 activation rows per workgroup tile (1, 2, 4 or 8); a workgroup owns 64 weight rows
    int kh;      // groups of four waves per workgroup, each on its share of K (2 with mbw < 4; 1 or 2 with mbw = 4; 1 with 8)
    int grid_n;  // tiles of 64 weight rows over all members: sum of ceil(N / 64)
    int grid_m;  // ceil(M / (16 mbw))
};

constexpr int kGemmtMaxGroup = 4;  // linears one launch can serve (they share x, K, M and w_bits)

// The linears of a launch.  Tiles of 64 weight rows are numbered through the members: member g owns tiles
// tile0[g] .. tile0[g + 1) (grid_n = tile0[count]).  Output rows of member g are ldo[g] elements apart (N[g] for a
// dense result; the sum of the N for results written side by side into one array).
struct GemmtMembers {
    const uint32_t *qweight[kGemmtMaxGroup];
    const uint16_t *lut[kGemmtMaxGroup];
    uint16_t *out[kGemmtMaxGroup];
    int N[kGemmtMaxGroup];
    int tile0[kGemmtMaxGroup + 1];
    int count;
    long long ldo[kGemmtMaxGroup];
};

// Launches gemmt_kbit_kernel<BITS, 1, geo.mbw, geo.kh> on `stream`.  K must be a multiple of 128.
template <int BITS>
void launch_gemmt(const GemmtGeometry &geo, const uint16_t *x, const GemmtMembers &members, int M, int K, hipStream_t stream);

extern template void launch_gemmt<3>(const GemmtGeometry &, const uint16_t *, const GemmtMembers &, int, int, hipStream_t);
extern template void launch_gemmt<4>(const GemmtGeometry &, const uint16_t *, const GemmtMembers &, int, int, hipStream_t);
extern template void launch_gemmt<5>(const GemmtGeometry &, const uint16_t *, const GemmtMembers &, int, int, hipStream_t);
extern template void launch_gemmt<6>(const GemmtGeometry &, const uint16_t *, const GemmtMembers &, int, int, hipStream_t);
extern template void launch_gemmt<7>(const GemmtGeometry &, const uint16_t *, const GemmtMembers &, int, int, hipStream_t);
extern template void launch_gemmt<8>(const GemmtGeometry &, const uint16_t *, const GemmtMembers &, int, int, hipStream_t);

}  // namespace ap

// Host-side launch interface of the 4x4x4 matrix-core skinny GEMM (one translation unit per
// bit-width: ap_gemv4_inst.hip with -DAP_BITS=b).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ap {

constexpr int kGemv4MaxSeg = 16;      // waves per workgroup, up to 4 activation rows
constexpr int kGemv4MaxSegTwo = 8;    // waves per workgroup, 5..8 activation rows

struct Gemv4Geometry {
    int mg;    // groups of four activation rows: 1 or 2
    int G;     // word groups (16 words of each of 4 rows) per wave: 1, 2 or 4 (mg = 2: 1 only)
    int S;     // waves per workgroup
    int rq;    // row quads per workgroup: 2 with mg = 1, 4 with mg = 2 (only those are instantiated)
    int grid;  // workgroups = ceil(N / (4 rq))
};

// Launches gemv4_kbit_kernel<BITS, 1, geo.G, 2, *> (1 <= M <= 4) or <BITS, 2, 1, 4, *> (5 <= M <= 8) on `stream`.
template <int BITS>
void launch_gemv4(const Gemv4Geometry &geo, const uint16_t *x, const uint32_t *qweight, const uint16_t *lut,
                  uint16_t *out, int M, int N, int K, hipStream_t stream);

extern template void launch_gemv4<3>(const Gemv4Geometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, int, hipStream_t);
extern template void launch_gemv4<4>(const Gemv4Geometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, int, hipStream_t);
extern template void launch_gemv4<5>(const Gemv4Geometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, int, hipStream_t);
extern template void launch_gemv4<6>(const Gemv4Geometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, int, hipStream_t);
extern template void launch_gemv4<7>(const Gemv4Geometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, int, hipStream_t);
extern template void launch_gemv4<8>(const Gemv4Geometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, int, hipStream_t);

}  // namespace ap

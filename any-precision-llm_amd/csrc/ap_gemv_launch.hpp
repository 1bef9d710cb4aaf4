// Host-side launch interface of the GEMV kernels.  The kernels of one bit-width are
// compiled in their own translation unit (ap_gemv_inst.hip with -DAP_BITS=b) so that the
// six bit-widths build in parallel; ap_capi.hip only sees these declarations.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ap {

constexpr int kGemvMaxSeg = 16;    // K-segments (waves) per workgroup
constexpr int kGemvMaxGroup = 4;   // linears one launch can serve (same x, K, M, w_bits)

// The linears of one launch.  Member g owns workgroups [wg_end[g-1], wg_end[g]); passed to the
// kernel by value (kernel arguments), so a launch needs no device-side descriptor.
struct GemvMembers {
    const uint32_t *qweight[kGemvMaxGroup];
    const uint16_t *lut[kGemvMaxGroup];
    uint16_t *out[kGemvMaxGroup];
    int n[kGemvMaxGroup];       // rows
    int wg_end[kGemvMaxGroup];  // first workgroup past the member
    int count;
};

struct GemvGeometry {
    int wpl;   // words per lane per plane (1 or 2)
    int S;     // K-segments = waves per workgroup
    int R;     // rows per workgroup (1 up to two activation rows, 2, or 4 up to four activation rows)
    int grid;  // workgroups (of all members together)
};

// Launches gemv_kbit_kernel<BITS, M, geo.wpl, geo.R, *> on `stream`.  1 <= M <= 8.
template <int BITS>
void launch_gemv(int M, const GemvGeometry &geo, const uint16_t *x, const GemvMembers &members, int K,
                 hipStream_t stream);

// Launches gemv_kbit_kernel<BITS, M, 1, 2, *, true>: members 0 and 1 of `members` are two linears of n[0] rows
// each (gate and up), out[0] receives silu(member 0) * member 1; geo.wpl = 1, geo.R = 2, geo.grid = n[0].  1 <= M <= 4.
template <int BITS>
void launch_gemv_pair(int M, const GemvGeometry &geo, const uint16_t *x, const GemvMembers &members, int K,
                      hipStream_t stream);

extern template void launch_gemv_pair<3>(int, const GemvGeometry &, const uint16_t *, const GemvMembers &, int, hipStream_t);
extern template void launch_gemv_pair<4>(int, const GemvGeometry &, const uint16_t *, const GemvMembers &, int, hipStream_t);
extern template void launch_gemv_pair<5>(int, const GemvGeometry &, const uint16_t *, const GemvMembers &, int, hipStream_t);
extern template void launch_gemv_pair<6>(int, const GemvGeometry &, const uint16_t *, const GemvMembers &, int, hipStream_t);
extern template void launch_gemv_pair<7>(int, const GemvGeometry &, const uint16_t *, const GemvMembers &, int, hipStream_t);
extern template void launch_gemv_pair<8>(int, const GemvGeometry &, const uint16_t *, const GemvMembers &, int, hipStream_t);

extern template void launch_gemv<3>(int, const GemvGeometry &, const uint16_t *, const GemvMembers &, int, hipStream_t);
extern template void launch_gemv<4>(int, const GemvGeometry &, const uint16_t *, const GemvMembers &, int, hipStream_t);
extern template void launch_gemv<5>(int, const GemvGeometry &, const uint16_t *, const GemvMembers &, int, hipStream_t);
extern template void launch_gemv<6>(int, const GemvGeometry &, const uint16_t *, const GemvMembers &, int, hipStream_t);
extern template void launch_gemv<7>(int, const GemvGeometry &, const uint16_t *, const GemvMembers &, int, hipStream_t);
extern template void launch_gemv<8>(int, const GemvGeometry &, const uint16_t *, const GemvMembers &, int, hipStream_t);

}  // namespace ap

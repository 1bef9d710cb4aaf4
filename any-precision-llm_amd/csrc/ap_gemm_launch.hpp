// Host-side launch interface of the fused dequant -> MFMA GEMM kernels (one translation
// unit per bit-width: ap_gemm_inst.hip with -DAP_BITS=b).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ap {

constexpr int kGemmMaxM = 128;    // activation rows one launch serves (8 MFMA row blocks)
constexpr int kGemmMaxSplit = 8;  // K-split waves per workgroup

struct GemmGeometry {
    int mb;    // activation row blocks of 16
    int ks;    // K-split waves per workgroup
    int rb;    // blocks of 16 weight rows per workgroup: 1, or 2 (only with K % 128 == 0 and mb <= 2)
    int grid;  // workgroups = ceil(N / (16 rb))
    int lookahead;  // 1: gathers one word ahead of the matrix instructions (one or two activation row blocks, rb = 1, K % 128 == 0)
};

// Launches gemm_kbit_kernel<BITS, geo.mb, ..., geo.rb> on `stream`.
template <int BITS>
void launch_gemm(const GemmGeometry &geo, const uint16_t *x, const uint32_t *qweight, const uint16_t *lut,
                 uint16_t *out, int M, int N, int K, hipStream_t stream);

extern template void launch_gemm<3>(const GemmGeometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, int, hipStream_t);
extern template void launch_gemm<4>(const GemmGeometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, int, hipStream_t);
extern template void launch_gemm<5>(const GemmGeometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, int, hipStream_t);
extern template void launch_gemm<6>(const GemmGeometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, int, hipStream_t);
extern template void launch_gemm<7>(const GemmGeometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, int, hipStream_t);
extern template void launch_gemm<8>(const GemmGeometry &, const uint16_t *, const uint32_t *, const uint16_t *, uint16_t *, int, int, int, hipStream_t);

}  // namespace ap

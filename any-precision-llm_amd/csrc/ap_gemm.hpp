// Fused bitplane dequant -> MFMA GEMM for gfx950, 1 <= M <= 128:
//     out[m,n] = sum_k x[m,k] * lut[n, index_b(n,k)]      (fp16 operands, fp32 accumulate)
//
// The reference has no fused kernel: above 8 activation rows it writes the whole fp16
// weight with dequant_kbit and calls torch.matmul
// (any_precision/modules/AnyPrecisionLinear.py:60-62).  For the batches a serving loop
// sees (tens of rows) that GEMM is bound by reading the fp16 weight it has just written;
// here the planes are read once (w_bits/16 of that traffic) and the dequantised weights
// never leave the register file.
//
// Mapping: v_mfma_f32_16x16x32_f16 wants, in lane l, eight consecutive-k halves of
// B[k][n] for n = l % 16 and k-group l / 16, and the same of A[m][k] for m = l % 16.  The
// packed layout hands out exactly such octets: byte group j of word w of row n holds
// eight consecutive elements, and words 4s..4s+3 of a chunk hold 32 consecutive ones.
// So lane l owns row n0 + l % 16 and word 4s + l / 16; it rebuilds the 32 indices of its
// word, gathers them from its row's table in LDS and has, for every byte group j, one
// B operand ready in registers -- no LDS round trip for the weights.  The matching A
// operand is x[m][k0 + 8 (l/16) .. +7]: 64 contiguous bytes per activation row.
//
// A workgroup is KS waves that share 16 weight rows and split K; their fp32 partial
// tiles meet in LDS and are added in a fixed order.  Plane loads are 4 bytes per lane
// (16 contiguous bytes per row and instruction); the 64-byte line they share is consumed
// by four consecutive steps of the same wave.
#pragma once
#include "ap_bitplane.hpp"
#include "ap_device.hpp"

namespace ap {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

constexpr int kGemmRows = 16;     // weight rows per workgroup (one MFMA column block)
constexpr int kGemmMaxSplit = 8;  // K-split waves per workgroup

// MB = activation row blocks of 16 (M <= 16*MB).  Grid: ceil(N/16) workgroups of (64, KS).
template <int BITS, int MB>
__global__ __launch_bounds__(kGemmMaxSplit *kWave) void gemm_kbit_kernel(
    const half_t *__restrict__ x, const uint32_t *__restrict__ qweight, const half_t *__restrict__ lut,
    half_t *__restrict__ out, int M, int N, int K) {
    constexpr int NC = 1 << BITS;
    __shared__ __attribute__((aligned(16))) half_t tables[kGemmRows][NC];
    __shared__ float red[kGemmMaxSplit][MB][4][kWave];

    const int lane = threadIdx.x;
    const int ks = __builtin_amdgcn_readfirstlane(threadIdx.y), KS = blockDim.y;
    const int col = lane & 15, grp = lane >> 4;
    const int W = K >> 5;
    const size_t plane_stride = (size_t)N * W;
    const int n0 = blockIdx.x * kGemmRows;
    const int row = min(n0 + col, N - 1);  // rows past N repeat row N-1 and are not stored

    // stage the 16 tables (16 * NC halves) with the whole workgroup
    {
        const int nthr = KS * kWave, tid = ks * kWave + lane;
        const uint32_t *src = reinterpret_cast<const uint32_t *>(lut);
        uint32_t *dst = reinterpret_cast<uint32_t *>(&tables[0][0]);
        for (int i = tid; i < kGemmRows * NC / 2; i += nthr) {
            const int r = i / (NC / 2), c = i - r * (NC / 2);
            dst[i] = src[(size_t)min(n0 + r, N - 1) * (NC / 2) + c];
        }
    }
    __syncthreads();
    const half_t *tab = tables[col];

    // this wave's range of 4-word steps
    const int steps = (W + 3) >> 2;
    const int s_begin = (int)((long long)steps * ks / KS), s_end = (int)((long long)steps * (ks + 1) / KS);

    float4_t acc[MB];
#pragma unroll
    for (int mb = 0; mb < MB; mb++) acc[mb] = float4_t{0.f, 0.f, 0.f, 0.f};

    const uint32_t *wrow = qweight + (size_t)row * W;
    auto fetch = [&](int step, uint32_t(&q)[BITS]) {
        const int w = min(4 * step + grp, W - 1);
#pragma unroll
        for (int p = 0; p < BITS; p++) q[p] = __builtin_nontemporal_load(wrow + p * plane_stride + w);
    };

    uint32_t qn[BITS];
    if (s_begin < s_end) fetch(s_begin, qn);
    for (int step = s_begin; step < s_end; step++) {
        uint32_t q[BITS];
#pragma unroll
        for (int p = 0; p < BITS; p++) q[p] = qn[p];
        if (step + 1 < s_end) fetch(step + 1, qn);

        const int w = 4 * step + grp;
        const bool live = w < W;            // words past the row end contribute zeros
        const int wc = live ? w : W - 1;

        uint32_t idx[8];
        planes_to_indices<BITS>(q, idx);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int sh = 8 * (3 - j);
            // B operand: the eight weights of byte group j
            u32x4 bw;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t lo = __builtin_bit_cast(uint16_t, tab[(idx[2 * i] >> sh) & 0xffu]);
                const uint32_t hi = __builtin_bit_cast(uint16_t, tab[(idx[2 * i + 1] >> sh) & 0xffu]);
                bw[i] = live ? (lo | (hi << 16)) : 0u;
            }
            const half8_t bfrag = __builtin_bit_cast(half8_t, bw);
            const int k0 = group_base(wc, j, K);
#pragma unroll
            for (int mb = 0; mb < MB; mb++) {
                const int m = min(mb * 16 + col, M - 1);  // rows past M repeat row M-1 and are not stored
                const half8_t afrag = *reinterpret_cast<const half8_t *>(x + (size_t)m * K + k0);
                acc[mb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(afrag, bfrag, acc[mb], 0, 0, 0);
            }
        }
    }

    // Combine the K-split partial tiles in wave order (also with one wave: it keeps the
    // accumulator indices static).  D[i][j]: lane l holds rows i = 4 (l / 16) + v, column l % 16.
#pragma unroll
    for (int mb = 0; mb < MB; mb++)
#pragma unroll
        for (int v = 0; v < 4; v++) red[ks][mb][v][lane] = acc[mb][v];
    __syncthreads();
    for (int t = ks; t < MB * 4; t += KS) {
        const int mb = t >> 2, v = t & 3;
        float sum = 0.f;
        for (int kk = 0; kk < KS; kk++) sum += red[kk][mb][v][lane];
        const int m = mb * 16 + 4 * grp + v;
        if (m < M && n0 + col < N) out[(size_t)m * N + n0 + col] = (half_t)sum;
    }
}

}  // namespace ap

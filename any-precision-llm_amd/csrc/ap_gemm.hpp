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
// tiles meet in LDS and are added in a fixed order.
//
// Plane loads: with VEC4 (K a multiple of 128) a lane loads the four words 16S + 4g .. +3
// of its row in one 16-byte load -- the four lanes of a row cover one 64-byte line -- and
// the words are then transposed across the four 16-lane rows of the wave
// (v_permlane32_swap / v_permlane16_swap) so that lane g holds words 16S + 4i + g,
// i = 0..3: at step i the four lanes of a row again hold four consecutive words.  Without
// VEC4 a lane loads one word per step (16 contiguous bytes per row and instruction) and
// the 64-byte line is re-read from L1/L2 by the next three steps.
#pragma once
#include "ap_bitplane.hpp"
#include "ap_device.hpp"

namespace ap {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

constexpr int kGemmRows = 16;     // weight rows per workgroup (one MFMA column block)
constexpr int kGemmMaxSplit = 8;  // K-split waves per workgroup

// 4x4 transpose of r[0..3] across the four 16-lane rows of the wave: on return r[i] of
// row g holds what r[g] of row i held.
__device__ __forceinline__ void transpose_rows4(uint32_t (&r)[4]) {
    auto a = __builtin_amdgcn_permlane32_swap(r[0], r[2], false, false);  // rows 2,3 of r0 <-> rows 0,1 of r2
    auto b = __builtin_amdgcn_permlane32_swap(r[1], r[3], false, false);
    auto c = __builtin_amdgcn_permlane16_swap(a[0], b[0], false, false);  // odd rows of r0 <-> even rows of r1
    auto d = __builtin_amdgcn_permlane16_swap(a[1], b[1], false, false);
    r[0] = c[0];
    r[1] = c[1];
    r[2] = d[0];
    r[3] = d[1];
}

// MB = activation row blocks of 16 (M <= 16*MB).  Grid: ceil(N/16) workgroups of (64, KS).
template <int BITS, int MB, bool VEC4>
__global__ __launch_bounds__(kGemmMaxSplit *kWave) void gemm_kbit_kernel(
    const half_t *__restrict__ x, const uint32_t *__restrict__ qweight, const half_t *__restrict__ lut,
    half_t *__restrict__ out, int M, int N, int K) {
    constexpr int NC = 1 << BITS;
    constexpr int WPS = VEC4 ? 4 : 1;  // words per lane and step
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
    // LDS byte address of this lane's table (LDS pointers are 32-bit offsets)
    typedef __attribute__((address_space(3))) half_t lds_half_t;
    const uint32_t tab_base = (uint32_t)(uintptr_t)((lds_half_t *)&tables[0][0]) + (uint32_t)col * (NC * 2);

    // this wave's range of steps (4 * WPS words of every row per step)
    const int steps = (W + 4 * WPS - 1) / (4 * WPS);
    const int s_begin = (int)((long long)steps * ks / KS), s_end = (int)((long long)steps * (ks + 1) / KS);

    float4_t acc[MB];
#pragma unroll
    for (int mb = 0; mb < MB; mb++) acc[mb] = float4_t{0.f, 0.f, 0.f, 0.f};

    const uint32_t *wrow = qweight + (size_t)row * W;
    // q[p][i]: plane p, i-th word of this lane for the step
    auto fetch = [&](int step, uint32_t(&q)[BITS][WPS]) {
        if constexpr (VEC4) {
            // W % 4 == 0: a quad is entirely inside the row or entirely past its end (then it is
            // clamped to the last quad and never used)
            const int w = min(16 * step + 4 * grp, W - 4);
#pragma unroll
            for (int p = 0; p < BITS; p++) {
                const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(wrow + p * plane_stride + w));
#pragma unroll
                for (int i = 0; i < 4; i++) q[p][i] = v[i];
            }
        } else {
            // plain (temporal) loads: the 64-byte line is needed again by the next three steps
            const int w = min(4 * step + grp, W - 1);
#pragma unroll
            for (int p = 0; p < BITS; p++) q[p][0] = wrow[p * plane_stride + w];
        }
    };

    uint32_t qn[BITS][WPS];
    if (s_begin < s_end) fetch(s_begin, qn);
    for (int step = s_begin; step < s_end; step++) {
        uint32_t q[BITS][WPS];
#pragma unroll
        for (int p = 0; p < BITS; p++)
#pragma unroll
            for (int i = 0; i < WPS; i++) q[p][i] = qn[p][i];
        if (step + 1 < s_end) fetch(step + 1, qn);
        if constexpr (VEC4) {
#pragma unroll
            for (int p = 0; p < BITS; p++) transpose_rows4(q[p]);
        }

        static_for<WPS>([&](auto i_c) {
            constexpr int wi = decltype(i_c)::value;
            const int w = 4 * (WPS * step + wi) + grp;
            const bool live = w < W;  // words past the row end contribute zeros
            const int wc = live ? w : W - 1;

            uint32_t qq[BITS];
#pragma unroll
            for (int p = 0; p < BITS; p++) qq[p] = q[p][wi];
            // index bytes hold the byte offset into the table (index * 2) where that fits a byte
            constexpr int PRE = BITS <= 7 ? 1 : 0;
            uint32_t idx[8];
            planes_to_indices<BITS, PRE>(qq, idx);
            static_for<4>([&](auto j_c) {
                constexpr int j = decltype(j_c)::value, c = 3 - j;
                // B operand: the eight weights of byte group j
                u32x4 bw;
                static_for<4>([&](auto e_c) {
                    constexpr int i = decltype(e_c)::value;
                    uint32_t a0, a1;
                    if constexpr (PRE) {
                        a0 = byte_add<c>(tab_base, idx[2 * i]);
                        a1 = byte_add<c>(tab_base, idx[2 * i + 1]);
                    } else {
                        a0 = tab_base + byte_offset<c, 1>(idx[2 * i]);
                        a1 = tab_base + byte_offset<c, 1>(idx[2 * i + 1]);
                    }
                    const uint32_t lo = *reinterpret_cast<const __attribute__((address_space(3))) uint16_t *>(a0);
                    const uint32_t hi = *reinterpret_cast<const __attribute__((address_space(3))) uint16_t *>(a1);
                    bw[i] = live ? (lo | (hi << 16)) : 0u;
                });
                const half8_t bfrag = __builtin_bit_cast(half8_t, bw);
                const int k0 = group_base(wc, j, K);
#pragma unroll
                for (int mb = 0; mb < MB; mb++) {
                    const int m = min(mb * 16 + col, M - 1);  // rows past M repeat row M-1 and are not stored
                    const half8_t afrag = *reinterpret_cast<const half8_t *>(x + (size_t)m * K + k0);
                    acc[mb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(afrag, bfrag, acc[mb], 0, 0, 0);
                }
            });
        });
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

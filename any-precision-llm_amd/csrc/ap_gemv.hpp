// Bitplane GEMV / skinny GEMM for gfx950, 1 <= M <= 8:
//     out[m,n] = sum_k x[m,k] * lut[n, index_b(n,k)]      (fp32 accumulate, fp16 out)
//
// Replaces the reference's matmul_kbit_32<maxm,bits,use_ksplit>
// (any_precision/modules/kernels/matmul.cuh:16-167); the reference sums in
// fp16, this kernel in fp32.
//
// Mapping (wave64): a workgroup is S x G waves.  Wave (s,g) owns K-segment s
// (64*WPL consecutive words of a row = 2048*WPL elements) of the rows of row
// group g.  The activations a lane needs never change from row to row, so
// they are loaded once into registers, already ordered the way the packed
// layout scatters elements (4 runs of 8 consecutive elements per word).  Per
// row a lane then streams WPL words per plane (one 4*WPL-byte load per plane,
// a wave covers 256*WPL contiguous bytes), rebuilds its indices in registers,
// gathers from the row's table in this wave's LDS slot and feeds
// v_dot2c_f32_f16.  Lane partials are summed with DPP; when S > 1 the S
// segment partials of a row meet in LDS and are added in a fixed order, so the
// result is deterministic.
#pragma once
#include "ap_bitplane.hpp"
#include "ap_device.hpp"

namespace ap {

constexpr int kGemvMaxWaves = 16;  // S * G upper bound (1024 threads)
constexpr int kGemvMaxRows = 8;    // rows per wave upper bound (R)

template <int WPL>
struct WordVec;
template <>
struct WordVec<1> { typedef uint32_t type; };
template <>
struct WordVec<2> { typedef u32x2 type; };
template <>
struct WordVec<4> { typedef u32x4 type; };

template <int WPL>
__device__ __forceinline__ uint32_t word_of(const typename WordVec<WPL>::type &v, int i) {
    if constexpr (WPL == 1) return v; else return v[i];
}

// Grid: ceil(N / (G*R)) workgroups of (64, S, G) threads.  Host guarantees
// W % WPL == 0, S*G*64 <= THREADS, R <= kGemvMaxRows, S*64*WPL >= W.
// THREADS (256, 512 or 1024) only bounds the workgroup size so that small
// workgroups may use more registers per lane (M x WPL x 16 of them hold x).
template <int BITS, int M, int WPL, int THREADS>
__global__ __launch_bounds__(THREADS) void gemv_kbit_kernel(
    const half_t *__restrict__ x, const uint32_t *__restrict__ qweight,
    const half_t *__restrict__ lut, half_t *__restrict__ out,
    int N, int K, int R) {
    constexpr int NC = 1 << BITS;
    typedef typename WordVec<WPL>::type wvec_t;
    constexpr int MAXW = THREADS / kWave;
    __shared__ __attribute__((aligned(16))) half_t tables[MAXW][2][NC];
    __shared__ float partial[MAXW * kGemvMaxRows * M];

    const int lane = threadIdx.x;
    const int s = threadIdx.y, S = blockDim.y;
    const int g = threadIdx.z, G = blockDim.z;
    const int wave = g * S + s;
    const int W = K >> 5;
    const size_t plane_stride = (size_t)N * W;

    const int w0 = (s * kWave + lane) * WPL;
    const bool valid = w0 < W;
    const int wl = valid ? w0 : 0;  // inactive lanes read word 0 and are zeroed below

    // Activations for this lane's words, in packed-layout order.
    u32x4 X[M][WPL][4];
#pragma unroll
    for (int m = 0; m < M; m++)
#pragma unroll
        for (int wi = 0; wi < WPL; wi++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const u32x4 v = *reinterpret_cast<const u32x4 *>(x + (size_t)m * K + group_base(wl + wi, j, K));
                X[m][wi][j] = valid ? v : u32x4{0u, 0u, 0u, 0u};
            }

    const int row0 = blockIdx.x * (G * R) + g;
    half_t(*tab)[NC] = tables[wave];

    auto fetch_planes = [&](int row, wvec_t(&q)[BITS]) {
        const uint32_t *p0 = qweight + (size_t)row * W + wl;
#pragma unroll
        for (int p = 0; p < BITS; p++) q[p] = *reinterpret_cast<const wvec_t *>(p0 + p * plane_stride);
    };

    wvec_t qn[BITS];
    LutRegs<BITS> ln;
    if (row0 < N) {
        fetch_planes(row0, qn);
        ln = lut_fetch<BITS>(lut + (size_t)row0 * NC, lane);
    }

    for (int r = 0; r < R; r++) {
        const int row = row0 + r * G;
        if (row >= N) break;  // uniform per wave
        wvec_t q[BITS];
#pragma unroll
        for (int p = 0; p < BITS; p++) q[p] = qn[p];
        lut_stage<BITS>(ln, tab[r & 1], lane);
        __builtin_amdgcn_wave_barrier();

        const int next = row + G;
        if (r + 1 < R && next < N) {
            fetch_planes(next, qn);
            ln = lut_fetch<BITS>(lut + (size_t)next * NC, lane);
        }

        const half_t *t = tab[r & 1];
        float acc[M];
#pragma unroll
        for (int m = 0; m < M; m++) acc[m] = 0.f;
#pragma unroll
        for (int wi = 0; wi < WPL; wi++) {
            uint32_t qq[BITS];
#pragma unroll
            for (int p = 0; p < BITS; p++) qq[p] = word_of<WPL>(q[p], wi);
            uint32_t idx[8];
            planes_to_indices<BITS>(qq, idx);
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int sh = 8 * (3 - j);
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const uint16_t lo = __builtin_bit_cast(uint16_t, t[(idx[2 * i] >> sh) & 0xffu]);
                    const uint16_t hi = __builtin_bit_cast(uint16_t, t[(idx[2 * i + 1] >> sh) & 0xffu]);
                    const uint32_t wpair = (uint32_t)lo | ((uint32_t)hi << 16);
#pragma unroll
                    for (int m = 0; m < M; m++) acc[m] = dot2(wpair, X[m][wi][j][i], acc[m]);
                }
            }
        }
#pragma unroll
        for (int m = 0; m < M; m++) {
            const float tot = wave_sum(valid ? acc[m] : 0.f);
            if (lane == 0) {
                if (S == 1) out[(size_t)m * N + row] = (half_t)tot;
                else partial[((g * kGemvMaxRows + r) * S + s) * M + m] = tot;
            }
        }
    }

    if (S > 1) {
        __syncthreads();
        const int tid = (g * S + s) * kWave + lane;
        const int nthreads = S * G * kWave;
        for (int i = tid; i < G * R * M; i += nthreads) {
            const int m = i % M, gr = i / M;
            const int rr = gr % R, gg = gr / R;
            const int row = blockIdx.x * (G * R) + rr * G + gg;
            if (row < N) {
                float tot = 0.f;
                for (int ss = 0; ss < S; ss++) tot += partial[((gg * kGemvMaxRows + rr) * S + ss) * M + m];
                out[(size_t)m * N + row] = (half_t)tot;
            }
        }
    }
}

}  // namespace ap

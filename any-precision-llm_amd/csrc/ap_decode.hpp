// The parts of a Llama-architecture decode step that sit between the bitplane linears, for ONE new
// token: residual add + RMSNorm, SiLU(gate) * up, and rotary embedding + key/value cache append +
// attention over the cache.  The reference has no kernels for them: its model wrapper calls the Hugging
// Face modules (any_precision/modules/AnyPrecisionForCausalLM.py:88-97), which at batch 1 cost a dozen
// launch-bound library kernels per layer between two GEMVs.  fp16 in memory, fp32 arithmetic, one rounding
// per output.
#pragma once
#include <math.h>

#include "ap_device.hpp"

namespace ap {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));

constexpr int kNormThreads = 256;
constexpr int kAttnThreads = 1024;  // sixteen waves: the kernel is a chain of load latencies, more waves = more loads in flight
constexpr int kAttnMaxLen = 8192;  // cache rows one launch can attend over (scores live in LDS)

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
    return v;
}

// One workgroup per row of H elements (H % 8 == 0):
//     s = h + delta (rounded to fp16, as an fp16 add; delta may be null), written to h_out;
//     x_out = s * rsqrt(mean(s^2) + eps) * weight.
// h_out may alias h.  Rows of up to 8 * kNormThreads * kNormHeld elements (8192) stay in registers between the
// two passes and the weight is requested before the reduction; longer rows re-read what they wrote.
constexpr int kNormHeld = 4;
__global__ __launch_bounds__(kNormThreads) void add_rmsnorm_kernel(const half_t *h, const half_t *delta,
                                                                   const half_t *__restrict__ weight, half_t *h_out,
                                                                   half_t *__restrict__ x_out, int H, float eps) {
    __shared__ float red[kNormThreads / kWave];
    const size_t row = blockIdx.x;
    const int tid = threadIdx.x;
    const half_t *hr = h + row * H;
    const half_t *dr = delta ? delta + row * H : nullptr;
    half_t *ho = h_out + row * H;
    const bool rewrite = dr != nullptr || ho != hr;
    constexpr int STEP = kNormThreads * 8;
    half8_t held[kNormHeld], wheld[kNormHeld];
    float ss = 0.f;
    auto summed = [&](int i) {
        half8_t a = *reinterpret_cast<const half8_t *>(hr + i);
        if (dr) {
            const half8_t b = *reinterpret_cast<const half8_t *>(dr + i);
#pragma unroll
            for (int e = 0; e < 8; e++) a[e] = (half_t)((float)a[e] + (float)b[e]);
        }
        if (rewrite) *reinterpret_cast<half8_t *>(ho + i) = a;
#pragma unroll
        for (int e = 0; e < 8; e++) ss += (float)a[e] * (float)a[e];
        return a;
    };
#pragma unroll
    for (int c = 0; c < kNormHeld; c++) {
        const int i = tid * 8 + c * STEP;
        if (i < H) {
            wheld[c] = *reinterpret_cast<const half8_t *>(weight + i);
            held[c] = summed(i);
        }
    }
    for (int i = tid * 8 + kNormHeld * STEP; i < H; i += STEP) summed(i);
    ss = wave_sum(ss);
    if ((tid & (kWave - 1)) == kSumLane) red[tid / kWave] = ss;
    __syncthreads();
    float total = 0.f;
#pragma unroll
    for (int w = 0; w < kNormThreads / kWave; w++) total += red[w];
    const float rs = rsqrtf(total / (float)H + eps);
    auto scaled = [&](const half8_t &a, const half8_t &w, int i) {
        half8_t y;
#pragma unroll
        for (int e = 0; e < 8; e++) y[e] = (half_t)((float)a[e] * rs * (float)w[e]);
        *reinterpret_cast<half8_t *>(x_out + row * H + i) = y;
    };
#pragma unroll
    for (int c = 0; c < kNormHeld; c++) {
        const int i = tid * 8 + c * STEP;
        if (i < H) scaled(held[c], wheld[c], i);
    }
    const half_t *src = rewrite ? ho : hr;  // every thread re-reads exactly what it wrote
    for (int i = tid * 8 + kNormHeld * STEP; i < H; i += STEP)
        scaled(*reinterpret_cast<const half8_t *>(src + i), *reinterpret_cast<const half8_t *>(weight + i), i);
}

// out = gate / (1 + exp(-gate)) * up over n elements (n % 8 == 0).
__global__ __launch_bounds__(256) void silu_mul_kernel(const half_t *__restrict__ gate, const half_t *__restrict__ up,
                                                       half_t *__restrict__ out, long long n) {
    const long long stride = (long long)gridDim.x * blockDim.x * 8;
    for (long long i = ((long long)blockIdx.x * blockDim.x + threadIdx.x) * 8; i < n; i += stride) {
        const half8_t g = *reinterpret_cast<const half8_t *>(gate + i);
        const half8_t u = *reinterpret_cast<const half8_t *>(up + i);
        half8_t y;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const float x = (float)g[e];
            y[e] = (half_t)(x / (1.f + __expf(-x)) * (float)u[e]);
        }
        *reinterpret_cast<half8_t *>(out + i) = y;
    }
}

// Greedy token selection and the bookkeeping of a decode step in one workgroup:
//     t = argmax(logits[0 .. n))  (the first index of the maximum; a NaN counts as the maximum, as torch.argmax has it);
//     p = *pos + 1; if p < max_len: emitted[p] = t, *pos = p;  *tok = t.
// Replaces an argmax reduction, an increment, an indexed store and a copy -- four launch-bound library kernels.
constexpr int kAdvanceThreads = 1024;
__global__ __launch_bounds__(kAdvanceThreads) void decode_advance_kernel(const half_t *__restrict__ logits, int n,
                                                                        long long *pos, long long *tok, long long *emitted,
                                                                        int max_len) {
    __shared__ float best_v[kAdvanceThreads / kWave];
    __shared__ int best_i[kAdvanceThreads / kWave];
    const int tid = threadIdx.x;
    // a > b in the order "NaN above everything, then by value, then the lower index"
    auto better = [](float av, int ai, float bv, int bi) {
        const bool an = av != av, bn = bv != bv;
        if (an != bn) return an;
        if (!an && av != bv) return av > bv;
        return ai < bi;
    };
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    const int nv = n / 8;  // whole 16-byte groups; the rest one by one
    constexpr int AHEAD = 4;  // 16-byte groups requested together: the scan is one chain of load latencies otherwise
    for (int g0 = tid; g0 < nv; g0 += AHEAD * kAdvanceThreads) {
        half8_t v[AHEAD];
#pragma unroll
        for (int a = 0; a < AHEAD; a++) {
            const int g = g0 + a * kAdvanceThreads;
            v[a] = reinterpret_cast<const half8_t *>(logits)[g < nv ? g : g0];
        }
#pragma unroll
        for (int a = 0; a < AHEAD; a++) {
            const int g = g0 + a * kAdvanceThreads;
            if (g < nv) {
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const float f = (float)v[a][e];
                    if (better(f, g * 8 + e, bv, bi)) {
                        bv = f;
                        bi = g * 8 + e;
                    }
                }
            }
        }
    }
    for (int i = nv * 8 + tid; i < n; i += kAdvanceThreads) {
        const float f = (float)logits[i];
        if (better(f, i, bv, bi)) {
            bv = f;
            bi = i;
        }
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        const float ov = __shfl_xor(bv, off, kWave);
        const int oi = __shfl_xor(bi, off, kWave);
        if (better(ov, oi, bv, bi)) {
            bv = ov;
            bi = oi;
        }
    }
    if ((tid & (kWave - 1)) == 0) {
        best_v[tid / kWave] = bv;
        best_i[tid / kWave] = bi;
    }
    __syncthreads();
    if (tid == 0) {
        for (int w = 1; w < kAdvanceThreads / kWave; w++)
            if (better(best_v[w], best_i[w], bv, bi)) {
                bv = best_v[w];
                bi = best_i[w];
            }
        const long long p = *pos + 1;
        if (p >= 0 && p < max_len) {
            emitted[p] = bi;
            *pos = p;
        }
        *tok = bi;
    }
}

// Attention of one new token at cache row pos = *pos_p, one workgroup per query head.
//   qkv     [n_heads + 2 n_kv_heads, HD]: the token's query, key and value heads before the rotary embedding
//   cosT, sinT [max_len, HD / 2] fp32: cos / sin of position * inverse frequency i
//   kcache, vcache [n_kv_heads, max_len, HD]: rows 0 .. pos-1 are read; row pos is written (rotated key, value)
//           by the first query head of each key/value group -- every workgroup uses its own copy of that row
//           from LDS, never the one in memory
//   out     [n_heads * HD]
// Rotary convention of the Hugging Face Llama model: x * cos + rotate_half(x) * sin with
// rotate_half(x) = (-x[HD/2:], x[:HD/2]).  Scores = (q . k) * scale, softmax and the weighted sum in fp32.
// A position outside 0 .. max_len-1 makes every workgroup return without touching memory.
template <int HD>
__global__ __launch_bounds__(kAttnThreads) void decode_attention_kernel(
    const half_t *__restrict__ qkv, const float *__restrict__ cosT, const float *__restrict__ sinT, half_t *kcache,
    half_t *vcache, const long long *__restrict__ pos_p, half_t *__restrict__ out, int nh, int nkv, int max_len,
    float scale) {
    constexpr int HALF = HD / 2;
    constexpr int DPL = HD / 4;    // score pass: four lanes share a key, DPL dims each
    constexpr int NCH = DPL / 8;   // 16-byte chunks of those
    constexpr int NW = kAttnThreads / kWave;
    constexpr int DPT = 8;                  // value pass: dims per lane (one 16-byte load)
    constexpr int LPK = HD / DPT;           // lanes per key
    constexpr int KPW = kWave / LPK;        // keys per wave and step
    static_assert(HD % 32 == 0 && HD <= 256 && LPK <= kWave, "");
    __shared__ float q_s[HD], kn_s[HD], vn_s[HD];
    __shared__ float sc[kAttnMaxLen];
    __shared__ float red[2][NW];
    __shared__ float ctx_s[NW * KPW][HD];

    const int head = blockIdx.x, tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const int group = nh / nkv, kvh = head / group;
    const bool writer = head % group == 0;
    const long long p64 = *pos_p;
    if (p64 < 0 || p64 >= max_len) return;  // uniform over the grid
    const int pos = (int)p64;

    // ---- rotary embedding of the query and the new key; the new row of the cache
    {
        const half_t *qr = qkv + (size_t)head * HD, *kr = qkv + (size_t)(nh + kvh) * HD;
        const half_t *vr = qkv + (size_t)(nh + nkv + kvh) * HD;
        half_t *kdst = kcache + ((size_t)kvh * max_len + pos) * HD, *vdst = vcache + ((size_t)kvh * max_len + pos) * HD;
        for (int i = tid; i < HALF; i += kAttnThreads) {
            const float c = cosT[(size_t)pos * HALF + i], s = sinT[(size_t)pos * HALF + i];
            const float q1 = (float)qr[i], q2 = (float)qr[i + HALF], k1 = (float)kr[i], k2 = (float)kr[i + HALF];
            q_s[i] = (q1 * c - q2 * s) * scale;
            q_s[i + HALF] = (q2 * c + q1 * s) * scale;
            const half_t a = (half_t)(k1 * c - k2 * s), b = (half_t)(k2 * c + k1 * s);
            kn_s[i] = (float)a;
            kn_s[i + HALF] = (float)b;
            if (writer) {
                kdst[i] = a;
                kdst[i + HALF] = b;
            }
        }
        for (int d = tid; d < HD; d += kAttnThreads) {
            const half_t v = vr[d];
            vn_s[d] = (float)v;
            if (writer) vdst[d] = v;
        }
    }
    __syncthreads();

    // ---- the first value rows this lane will need are requested now: they do not depend on the scores, and the
    // score pass and the softmax then hide their latency (LPK lanes per key, 8 dims = 16 bytes each)
    constexpr int PF = 6;  // steps of NW * KPW keys held in registers (384 keys at HD = 128); later ones load in place
    const int dl = lane % LPK, sub = lane / LPK;
    const half_t *vbase = vcache + (size_t)kvh * max_len * HD + dl * DPT;
    half8_t vpre[PF];
#pragma unroll
    for (int it = 0; it < PF; it++) {
        const int j = wave * KPW + sub + it * NW * KPW;
        vpre[it] = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
        if (j < pos) vpre[it] = *reinterpret_cast<const half8_t *>(vbase + (size_t)j * HD);
    }

    // ---- scores against the cached keys: four lanes per key
    {
        const int quad = tid >> 2, part = tid & 3;
        float qreg[DPL];
#pragma unroll
        for (int d = 0; d < DPL; d++) qreg[d] = q_s[part * DPL + d];
        const half_t *kbase = kcache + (size_t)kvh * max_len * HD + part * DPL;
#pragma unroll 4
        for (int j0 = 0; j0 < pos; j0 += kAttnThreads / 4) {
            const int j = j0 + quad;
            float s = 0.f;
            if (j < pos) {
                const u32x4 *p = reinterpret_cast<const u32x4 *>(kbase + (size_t)j * HD);
#pragma unroll
                for (int c = 0; c < NCH; c++) {
                    const u32x4 v = p[c];
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const uint32_t w = v[e];  // a copy: bit-casting the vector element itself reads element 0
                        const half2_t h2 = __builtin_bit_cast(half2_t, w);
                        s += (float)h2.x * qreg[c * 8 + 2 * e] + (float)h2.y * qreg[c * 8 + 2 * e + 1];
                    }
                }
            }
            s = dpp_add<0xB1>(s);  // the four lanes of a key
            s = dpp_add<0x4E>(s);
            if (part == 0 && j < pos) sc[j] = s;
        }
        if (tid < kWave) {  // the new key, from LDS
            float s = 0.f;
            for (int d = tid; d < HD; d += kWave) s += q_s[d] * kn_s[d];
            s = wave_sum(s);
            if (tid == kSumLane) sc[pos] = s;
        }
    }
    __syncthreads();

    // ---- softmax over rows 0 .. pos
    const int n = pos + 1;
    float m = -INFINITY;
    for (int j = tid; j < n; j += kAttnThreads) m = fmaxf(m, sc[j]);
    m = wave_max(m);
    if (lane == 0) red[0][wave] = m;
    __syncthreads();
    m = red[0][0];
#pragma unroll
    for (int w = 1; w < NW; w++) m = fmaxf(m, red[0][w]);
    float l = 0.f;
    for (int j = tid; j < n; j += kAttnThreads) {
        const float p = __expf(sc[j] - m);
        sc[j] = p;
        l += p;
    }
    l = wave_sum(l);
    if (lane == kSumLane) red[1][wave] = l;
    __syncthreads();  // also: every probability is in LDS
    l = 0.f;
#pragma unroll
    for (int w = 0; w < NW; w++) l += red[1][w];

    // ---- weighted sum of the values
    {
        float acc[DPT];
#pragma unroll
        for (int e = 0; e < DPT; e++) acc[e] = 0.f;
#pragma unroll
        for (int it = 0; it < PF; it++) {  // the prefetched rows (zeros past pos, and a zero weight past n)
            const int j = wave * KPW + sub + it * NW * KPW;
            const float p = j < n ? sc[j] : 0.f;
            if (j == pos) {
#pragma unroll
                for (int e = 0; e < DPT; e++) acc[e] += p * vn_s[dl * DPT + e];
            } else {
#pragma unroll
                for (int e = 0; e < DPT; e++) acc[e] += p * (float)vpre[it][e];
            }
        }
#pragma unroll 4
        for (int j = wave * KPW + sub + PF * NW * KPW; j < n; j += NW * KPW) {
            const float p = sc[j];
            if (j < pos) {
                const half8_t v = *reinterpret_cast<const half8_t *>(vbase + (size_t)j * HD);
#pragma unroll
                for (int e = 0; e < DPT; e++) acc[e] += p * (float)v[e];
            } else {
#pragma unroll
                for (int e = 0; e < DPT; e++) acc[e] += p * vn_s[dl * DPT + e];
            }
        }
#pragma unroll
        for (int e = 0; e < DPT; e++) ctx_s[wave * KPW + sub][dl * DPT + e] = acc[e];
    }
    __syncthreads();
    for (int d = tid; d < HD; d += kAttnThreads) {
        float s = 0.f;
#pragma unroll 8
        for (int r = 0; r < NW * KPW; r++) s += ctx_s[r][d];
        out[(size_t)head * HD + d] = (half_t)(s / l);
    }
}

}  // namespace ap

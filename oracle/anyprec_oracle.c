/*
 * CPU oracle for the any-precision bitplane path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C, the algorithm of the reference's packed
 * layout, bit transpose, dequant kernel and GEMV kernel.  It is the checker
 * the HIP kernels are compared against; it is never part of the shipped
 * library and nothing outside the test-suite, the smoke check and the
 * benchmark's CPU-baseline leg may call it.
 *
 * Reference sources restated (paths relative to the reference checkout):
 *   any_precision/quantization/pack.py:12-76,90-99      layout written to disk
 *   any_precision/modules/kernels/dequant.cuh:10-175    per-lane bit transpose
 *   any_precision/modules/kernels/dequant.cuh:177-242   dequant_kbit_store
 *   any_precision/modules/kernels/matmul.cuh:16-167     matmul_kbit_32
 *   any_precision/modules/kernels/main.cu:60-143        shapes, M, dispatch
 *   any_precision/evaluate/eval.py:104-105              index = code >> (P - b)
 *
 * Parity pins (all in tests/test_oracle_*.py):
 *   apo_pack_bitplanes   - hand-derived known answers (K=32, K=64), numpy
 *                          packbits+argsort statement of pack.py, and the
 *                          pack->dequant identity below.
 *   apo_transpose        - brute force over all codes x 32 bit positions
 *                          against the definition "index = top b bits".
 *   apo_dequant_kbit     - pack (follows pack.py) then dequant (follows the
 *                          kernel's addressing) must equal lut[code >> (P-b)]
 *                          (eval.py:104-105); two independent reference
 *                          sources have to agree for that to hold.
 *   apo_matmul_kbit      - one-hot x gives a dequant column, constant LUT
 *                          gives sum(x)*c, float64 numpy matmul on the
 *                          dequantised weights, linearity in x.
 * The reference accumulates the GEMV in fp16; this oracle accumulates in
 * double and rounds once to fp16, which is what the HIP path (fp32
 * accumulate) is compared with at 1e-2 relative tolerance.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define APO_WARP 32           /* lanes per warp in the reference kernels   */
#define APO_CHUNK_WORDS 32    /* words per full chunk (= one warp load)     */
#define APO_CHUNK_ELEMS 1024  /* K elements per full chunk                  */

/* ---- fp16 <-> fp32 (IEEE binary16, round-to-nearest-even) -------------- */

float apo_half_to_float(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else {                      /* subnormal: renormalise */
            int e = -1;
            do { man <<= 1; e++; } while (!(man & 0x400u));
            man &= 0x3ffu;
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

uint16_t apo_double_to_half(double d)
{
    /* One rounding, double -> binary16, ties to even. */
    if (isnan(d)) return 0x7e00u;
    uint16_t sign = signbit(d) ? 0x8000u : 0;
    double a = fabs(d);
    if (a >= 65520.0) return sign | 0x7c00u;          /* overflow to inf */
    if (a < 5.9604644775390625e-8 * 0.5) return sign; /* below half of min subnormal */
    int e;
    double m = frexp(a, &e);          /* a = m * 2^e, m in [0.5,1) */
    int exp16 = e - 1 + 15;           /* biased exponent if normal */
    double scaled;
    if (exp16 >= 1) {
        scaled = ldexp(m, 11);        /* 11 significant bits, in [1024,2048) */
    } else {
        scaled = ldexp(a, 24);        /* subnormal: units of 2^-24 */
        exp16 = 0;
    }
    double r = nearbyint(scaled);     /* default rounding mode = ties-to-even */
    uint32_t q = (uint32_t)r;
    if (exp16 >= 1) {
        if (q == 2048u) { q = 1024u; exp16++; }
        if (exp16 >= 31) return sign | 0x7c00u;
        return sign | (uint16_t)(exp16 << 10) | (uint16_t)(q - 1024u);
    }
    /* subnormal (q may reach 1024 -> smallest normal, encoding is continuous) */
    return sign | (uint16_t)q;
}

/* ---- layout: pack.py ---------------------------------------------------- */

/* pack.py:51-68 (_calculate_new_indices): destination byte of source byte
 * `idx` inside a group of `threads` lanes x 4 bytes.  */
static int apo_new_byte_index(int idx, int threads)
{
    int bytes_per_warp = threads * 4;
    int warp = idx / bytes_per_warp;
    int within = idx % bytes_per_warp;
    int lane = idx % threads;
    int byte_in_lane = (within / threads) ^ 3;   /* endianness flip */
    return warp * bytes_per_warp + lane * 4 + byte_in_lane;
}

/* pack.py:90-99 + 12-76.  codes: [N,K] uint8 (values < 2^P); qweight:
 * [P,N,K/32] uint32 (the int32 tensor's bit pattern).  K % 32 == 0. */
int apo_pack_bitplanes(const uint8_t *codes, int N, int K, int P, uint32_t *qweight)
{
    if (K % 32 != 0 || P < 1 || P > 8 || N < 0) return -1;
    int total_bytes = K / 8;
    int full = (total_bytes / 128) * 128;       /* bytes in full warps   */
    int rem = total_bytes - full;               /* bytes in the tail      */
    int rem_threads = rem / 4;
    uint8_t *src = (uint8_t *)malloc((size_t)total_bytes);
    uint8_t *dst = (uint8_t *)malloc((size_t)total_bytes);
    if (!src || !dst) { free(src); free(dst); return -2; }
    int W = K / 32;
    for (int p = 0; p < P; p++) {
        int bit = P - 1 - p;                    /* plane 0 = MSB (pack.py:92-96) */
        for (int n = 0; n < N; n++) {
            const uint8_t *row = codes + (size_t)n * K;
            /* np.packbits: first element lands in the byte's MSB */
            for (int b = 0; b < total_bytes; b++) {
                unsigned v = 0;
                for (int e = 0; e < 8; e++)
                    v = (v << 1) | ((row[b * 8 + e] >> bit) & 1u);
                src[b] = (uint8_t)v;
            }
            /* permuted = bitmaps[argsort(new_idx)]  <=>  permuted[new_idx[i]] = bitmaps[i] */
            for (int b = 0; b < full; b++)
                dst[apo_new_byte_index(b, APO_WARP)] = src[b];
            for (int b = 0; b < rem; b++)
                dst[full + apo_new_byte_index(b, rem_threads)] = src[full + b];
            /* reshape(-1,4).view(int32): little-endian words */
            uint32_t *out = qweight + ((size_t)p * N + n) * W;
            for (int w = 0; w < W; w++)
                out[w] = (uint32_t)dst[4 * w] | ((uint32_t)dst[4 * w + 1] << 8) |
                         ((uint32_t)dst[4 * w + 2] << 16) | ((uint32_t)dst[4 * w + 3] << 24);
        }
    }
    free(src); free(dst);
    return 0;
}

/* ---- per-lane bit transpose: dequant.cuh:10-175 ------------------------- */

/* q[0..bits-1]: one word per plane (plane 0 most significant).  q_w[e],
 * e = 0..7: byte c of q_w[e] is the `bits`-bit index of the element stored
 * at word bit 8c + (7 - e).  Equivalent to dequant<bits,false>. */
void apo_transpose(const uint32_t *q, int bits, uint32_t q_w[8])
{
    for (int e = 0; e < 8; e++) {
        uint32_t w = 0;
        for (int c = 0; c < 4; c++) {
            uint32_t idx = 0;
            for (int p = 0; p < bits; p++)
                idx = (idx << 1) | ((q[p] >> (8 * c + 7 - e)) & 1u);
            w |= idx << (8 * c);
        }
        q_w[e] = w;
    }
}

/* dequant<3,true> / dequant<4,true> (dequant.cuh:13-30,56-67): byte c of
 * q_w[m], m = 0..3, is (index(e=m) << bits) | index(e=m+4). */
void apo_transpose_pair(const uint32_t *q, int bits, uint32_t q_w[4])
{
    uint32_t s[8];
    apo_transpose(q, bits, s);
    for (int m = 0; m < 4; m++)
        q_w[m] = (s[m] << bits) | s[m + 4];
}

/* ---- dequant kernel: dequant.cuh:177-242 -------------------------------- */

/* W: [>=bits, N, K/32] uint32, C: [N, 2^bits] fp16 bits, O: [N,K] fp16 bits.
 * Walks exactly as the kernel does: row <-> warp, chunk i of 32 words,
 * lane t, tail chunk with eff = (K % 1024) / 32 lanes. */
int apo_dequant_kbit(const uint32_t *W, int N, int K, int bits,
                     const uint16_t *C, uint16_t *O)
{
    if (K % 32 != 0 || bits < 1 || bits > 8) return -1;
    const int words = K / 32;
    const int nc = 1 << bits;
    const int maxi = (K + APO_CHUNK_ELEMS - 1) / APO_CHUNK_ELEMS;
#pragma omp parallel for schedule(static)
    for (int row = 0; row < N; row++) {
        const uint16_t *lut = C + (size_t)row * nc;
        for (int i = 0; i < maxi; i++) {
            int eff = APO_WARP;
            if (i == K / APO_CHUNK_ELEMS) eff = (K % APO_CHUNK_ELEMS) / 32;
            for (int t = 0; t < eff; t++) {
                uint32_t q[8], q_w[8];
                for (int j = 0; j < bits; j++)
                    q[j] = W[((size_t)j * N + row) * words + (size_t)i * 32 + t];
                apo_transpose(q, bits, q_w);
                /* dequant.cuh:226-240: low byte first <-> j = 3; dq_w[4j+k] =
                 * (w[e=2k], w[e=2k+1]); store 8 halves at
                 * row*K + 8*eff*j + 1024*i + 8*t. */
                for (int j = 3; j >= 0; j--) {
                    uint16_t *dst = O + (size_t)row * K + 8 * eff * j + (size_t)i * APO_CHUNK_ELEMS + 8 * t;
                    for (int e = 0; e < 8; e++) {
                        dst[e] = lut[q_w[e] & 0xffu];
                        q_w[e] >>= 8;
                    }
                }
            }
        }
    }
    return 0;
}

/* ---- GEMV kernel: matmul.cuh:16-167 ------------------------------------- */

/* I: [M,K] fp16 bits, W as above, C: [N,2^bits], O: [M,N] fp16 bits.
 * Same walk as the kernel (chunks, tail, lane t, byte-group j, x offset
 * (l*K/8 + eff*j + i*128 + t) float4s = 8 halves each, matmul.cuh:123), but
 * the sum is carried in double and rounded once; Od (optional, may be NULL)
 * receives the unrounded sums. */
int apo_matmul_kbit(const uint16_t *I, const uint32_t *W, int M, int N, int K,
                    int bits, const uint16_t *C, uint16_t *O, double *Od)
{
    if (K % 32 != 0 || bits < 1 || bits > 8 || M < 1) return -1;
    const int words = K / 32;
    const int nc = 1 << bits;
    const int maxi = (K + APO_CHUNK_ELEMS - 1) / APO_CHUNK_ELEMS;
    float *xf = (float *)malloc(sizeof(float) * (size_t)M * K);
    if (!xf) return -2;
    for (size_t i = 0; i < (size_t)M * K; i++) xf[i] = apo_half_to_float(I[i]);
#pragma omp parallel for schedule(static)
    for (int row = 0; row < N; row++) {
        float lutf[256];
        for (int c = 0; c < nc; c++) lutf[c] = apo_half_to_float(C[(size_t)row * nc + c]);
        double acc[64];
        double *accp = acc;
        double *heap = NULL;
        if (M > 64) { heap = (double *)calloc((size_t)M, sizeof(double)); accp = heap; }
        for (int l = 0; l < M; l++) accp[l] = 0.0;
        for (int i = 0; i < maxi; i++) {
            int eff = APO_WARP;
            if (i == K / APO_CHUNK_ELEMS) eff = (K % APO_CHUNK_ELEMS) / 32;
            for (int t = 0; t < eff; t++) {
                uint32_t q[8], q_w[8];
                for (int j = 0; j < bits; j++)
                    q[j] = W[((size_t)j * N + row) * words + (size_t)i * 32 + t];
                apo_transpose(q, bits, q_w);
                for (int j = 3; j >= 0; j--) {
                    size_t xoff = (size_t)8 * ((size_t)eff * j + (size_t)i * 128 + t);
                    for (int e = 0; e < 8; e++) {
                        double w = (double)lutf[q_w[e] & 0xffu];
                        for (int l = 0; l < M; l++)
                            accp[l] += w * (double)xf[(size_t)l * K + xoff + e];
                        q_w[e] >>= 8;
                    }
                }
            }
        }
        for (int l = 0; l < M; l++) {
            if (O) O[(size_t)l * N + row] = apo_double_to_half(accp[l]);
            if (Od) Od[(size_t)l * N + row] = accp[l];
        }
        free(heap);
    }
    free(xf);
    return 0;
}

/* ---- CPU baseline variant: same semantics, arranged for host speed ------ */

/* Dequantise a row into fp32 (unpack + LUT gather), then M fp32 dot
 * products; threads over rows.  This is what the benchmark times as the
 * "reference semantics on CPU" leg (unpack + gather + matmul). */
int apo_matmul_kbit_fast(const uint16_t *I, const uint32_t *W, int M, int N, int K,
                         int bits, const uint16_t *C, uint16_t *O)
{
    if (K % 32 != 0 || bits < 1 || bits > 8 || M < 1) return -1;
    const int words = K / 32;
    const int nc = 1 << bits;
    const int full_chunks = K / APO_CHUNK_ELEMS;
    float *xf = (float *)malloc(sizeof(float) * (size_t)M * K);
    if (!xf) return -2;
    for (size_t i = 0; i < (size_t)M * K; i++) xf[i] = apo_half_to_float(I[i]);
#pragma omp parallel
    {
        float *wrow = (float *)malloc(sizeof(float) * (size_t)K);
#pragma omp for schedule(static)
        for (int row = 0; row < N; row++) {
            float lutf[256];
            for (int c = 0; c < nc; c++) lutf[c] = apo_half_to_float(C[(size_t)row * nc + c]);
            for (int w = 0; w < words; w++) {
                int i = w / 32, t = w % 32;
                int eff = (i == full_chunks) ? (K % APO_CHUNK_ELEMS) / 32 : APO_WARP;
                uint32_t q[8];
                for (int j = 0; j < bits; j++)
                    q[j] = W[((size_t)j * N + row) * words + w];
                for (int j = 0; j < 4; j++) {
                    float *dst = wrow + (size_t)i * APO_CHUNK_ELEMS + 8 * (eff * j + t);
                    int sh = 8 * (3 - j) + 7;
                    for (int e = 0; e < 8; e++) {
                        unsigned idx = 0;
                        for (int p = 0; p < bits; p++)
                            idx = (idx << 1) | ((q[p] >> (sh - e)) & 1u);
                        dst[e] = lutf[idx];
                    }
                }
            }
            for (int l = 0; l < M; l++) {
                const float *x = xf + (size_t)l * K;
                float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
                for (int k = 0; k < K; k += 4) {
                    s0 += wrow[k] * x[k];
                    s1 += wrow[k + 1] * x[k + 1];
                    s2 += wrow[k + 2] * x[k + 2];
                    s3 += wrow[k + 3] * x[k + 3];
                }
                O[(size_t)l * N + row] = apo_double_to_half((double)((s0 + s1) + (s2 + s3)));
            }
        }
        free(wrow);
    }
    free(xf);
    return 0;
}

int apo_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

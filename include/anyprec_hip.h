/*
 * libanyprec_hip -- C ABI of the MI355X (gfx950) any-precision bitplane kernels.
 *
 * Drop-in boundary for the reference's native ops module `any_precision_ext`
 * (any_precision/modules/kernels/main.cu).  Plain pointers and sizes only; all
 * pointers are device pointers on the current HIP device, all buffers are
 * owned by the caller, nothing is allocated or synchronised inside, and every
 * launch goes to the stream that is passed in (NULL = default stream).  The only
 * state the library keeps is the table of tuning knobs behind ap_set_tuning and
 * the CU count of each device, looked up on first use.
 *
 * Data formats (identical to the reference checkpoint format):
 *   qweight  uint32 [planes >= w_bits, N, K/32], contiguous; bit pattern of the
 *            int32 tensor written by any_precision/quantization/pack.py:90-99.
 *            Plane 0 is the MSB of the parent code; only planes 0..w_bits-1
 *            are read.
 *   lut      fp16 [N, 2^w_bits], the table for that w_bits
 *            (any_precision/modules/AnyPrecisionLinear.py:34-38).
 *   x        fp16 [M, K] row-major;  out fp16 [M, N] (matmul) or [N, K] (dequant).
 *
 * Return value: AP_OK (0), a negative AP_E* argument error, or a positive
 * hipError_t from the launch (an error some earlier HIP call of the thread left
 * behind is discarded, not reported).  An entry point that issues several launches
 * (grouped linears, batches split in chunks) stops at the first one that fails: the
 * outputs of the launches before it may already be written.  The library never exits the process (the
 * reference prints and calls exit(), main.cu:5-12).
 */
#ifndef ANYPREC_HIP_H
#define ANYPREC_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define AP_ABI_VERSION 8

enum {
    AP_OK = 0,
    AP_ENULL = -1,   /* a required pointer is NULL                          */
    AP_EBITS = -2,   /* w_bits outside 3..8 (main.cu:70,108)                */
    AP_ESHAPE = -3,  /* N < 1, K < 32 or K not a multiple of 32 (pack.py:15) */
    AP_EALIGN = -4,  /* a pointer is not 16-byte aligned                    */
    AP_EBATCH = -5,  /* M outside the range the entry point serves          */
    AP_ELIMIT = -6,  /* a size exceeds what the launch geometry can express */
    AP_EKNOB = -7    /* ap_set_tuning / ap_get_tuning: no knob of that name  */
};

/* Replaces dequant_kbit(qweight, lut, w_bits) -> Tensor[N,K]
 * (main.cu:60-91, kernel dequant.cuh:177-242).
 * out[n,k] = lut[n, code[n,k] >> (P - w_bits)], bit-exact copy of table entries. */
int ap_dequant_kbit(const uint32_t *qweight, const uint16_t *lut, uint16_t *out,
                    int N, int K, int w_bits, void *stream);

/* ap_dequant_kbit for `count` (1..8) linears of any shapes at one w_bits in ONE launch:
 * out[g][N[g], K[g]] = dequant(qweight[g], lut[g]).  The arrays are host arrays of `count` device
 * pointers / sizes.  For dequantising a whole decoder layer (seven linears) or a whole checkpoint
 * (config "full weight set"): the reference launches dequant_kbit_store once per linear
 * (main.cu:82-84); here the 64-word segments of all members share one grid, so the fixed cost and
 * the tail of a launch are paid once.  Results are bit-identical to `count` calls of ap_dequant_kbit.
 * AP_ELIMIT for count outside 1..8. */
int ap_dequant_kbit_group(int count, const uint32_t *const *qweight, const uint16_t *const *lut,
                          uint16_t *const *out, const int *N, const int *K, int w_bits, void *stream);

/* Replaces matmul_kbit(in, qweight, lut, w_bits) -> Tensor[..., N]
 * (main.cu:93-143, kernel matmul.cuh:16-167).  1 <= M <= 8 as in the
 * reference (main.cu:108).  fp32 accumulation, fp16 result. */
int ap_matmul_kbit(const uint16_t *x, const uint32_t *qweight, const uint16_t *lut,
                   uint16_t *out, int M, int N, int K, int w_bits, void *stream);

/* The GEMVs of `count` (1..4) linears that share x, M, K and w_bits:
 * out[g][M, N[g]] = x[M,K] . dequant(qweight[g], lut[g])^T, in ONE launch wherever the dot-product
 * kernel serves the set (always up to 4 activation rows; at 5..8 rows for sets with narrow members and
 * some 5-8-bit cases, see ap_matmul_kbit_group_route), otherwise member by member exactly as
 * ap_matmul_kbit would run each.  The arrays are host arrays of `count` device pointers / row counts.
 * For the q/k/v and gate/up projections of a decoder layer, whose launches are otherwise bound by the
 * fixed cost of a kernel launch.  No counterpart in the reference (its hook for it, fuse_layers, is a
 * stub: AnyPrecisionForCausalLM.py:168-172).  Results equal `count` calls of ap_matmul_kbit within
 * the 1e-2 bar of the path, and bit for bit whenever the same kernel serves both (always with the
 * tuning knobs gemv_stream, gemv_fine and matmul_mfma4 at 0: some shapes otherwise go to a kernel that
 * sums in another order when called one by one).  1 <= M <= 8. */
int ap_matmul_kbit_group(const uint16_t *x, int count, const uint32_t *const *qweight,
                         const uint16_t *const *lut, uint16_t *const *out, const int *N,
                         int M, int K, int w_bits, void *stream);

/* The gate and up projections of a SwiGLU MLP with their activation function, for 1 <= M <= 4 rows:
 *     out[M,N] = silu(x . W_gate^T) * (x . W_up^T),   silu(v) = v / (1 + exp(-v)),
 * two linears of equal shape [N,K] at the same w_bits, one launch, one rounding (fp32 until the store).
 * The reference computes the two products with two matmul_kbit calls (main.cu:93-143) and leaves the
 * activation to the Hugging Face MLP module it wraps (AnyPrecisionForCausalLM.py:88-97); its own
 * fuse_layers hook is a stub (:168-172).  AP_EBATCH beyond 4 rows, AP_ELIMIT for rows longer than
 * 32768 elements: call ap_matmul_kbit_group and ap_silu_mul there. */
int ap_matmul_kbit_swiglu(const uint16_t *x, const uint32_t *qweight_gate, const uint16_t *lut_gate,
                          const uint32_t *qweight_up, const uint16_t *lut_up, uint16_t *out,
                          int M, int N, int K, int w_bits, void *stream);

/* Fused dequant -> MFMA GEMM, M >= 1: out[M,N] = x[M,K] . dequant(qweight, lut)^T
 * without materialising the fp16 weight.  No single counterpart in the reference: it is the
 * M > 8 branch of AnyPrecisionLinear.forward (AnyPrecisionLinear.py:60-62: dequant_kbit,
 * main.cu:60-91, then torch.matmul) fused.  Two kernels: up to 128 activation rows a K-split
 * kernel with the weights of 16 rows in registers (more than 32 rows may run as launches of 32
 * each); from 81 rows on, and from 9..65 rows on where it measured faster, a tiled kernel whose
 * workgroups own 64 weight rows x 16..128 activation rows (the narrower the fewer tiles the grid
 * has) for the whole of K, ONE launch for any M (it needs K % 128 == 0; other row lengths go through the K-split kernel in chunks of 128 rows,
 * in order, on the same stream).  Correct for every M; faster than dequant + a library GEMM up to
 * about 256 rows at 3 bits and 64..128 rows at more bits -- beyond that use that pair.
 * fp32 accumulation, fp16 result. */
int ap_gemm_kbit(const uint16_t *x, const uint32_t *qweight, const uint16_t *lut,
                 uint16_t *out, int M, int N, int K, int w_bits, void *stream);

/* ap_gemm_kbit for 1..4 linears that share x, K and w_bits (the q/k/v or gate/up projections of a decoder
 * layer on a batch of rows): out[g][M, N[g]] = x[M,K] . dequant(qweight[g], lut[g])^T.  Where the tiled
 * kernel serves the set (K % 128 == 0) and pays -- more than 32 rows, or more than 8 where no member
 * has more than 8192 rows -- ONE launch whose tiles of 64 weight rows run through the members -- three 4096 x 4096 projections at 128 rows fill
 * the chip that one of them leaves half idle; otherwise one ap_gemm_kbit per member, in order.
 * ldo (may be NULL: dense results) gives the distance in elements between consecutive rows of each
 * out[g], so that the results can be written side by side into one [M, sum N] array (out[g] = its
 * column offset, ldo[g] = sum N); results that are not dense need the tiled kernel: AP_ESHAPE if
 * K % 128 != 0 then, AP_ELIMIT if M * K exceeds its 32-bit offsets (ask for dense results instead).  No counterpart in the reference (its fuse_layers hook is a stub,
 * AnyPrecisionForCausalLM.py:168-172).  AP_ELIMIT for count outside 1..4. */
int ap_gemm_kbit_group(const uint16_t *x, int count, const uint32_t *const *qweight,
                       const uint16_t *const *lut, uint16_t *const *out, const int *N,
                       const long long *ldo, int M, int K, int w_bits, void *stream);

/* Where the fused GEMM is the faster way to compute x . dequant(W)^T, from this library's measurements on
 * MI355X: ap_gemm_kbit_pays returns 1 if ap_gemm_kbit beats ap_dequant_kbit + a library fp16 GEMM for M
 * activation rows on an [N, K] linear at w_bits, 0 if the pair wins (the reference always takes the pair
 * above 8 rows, AnyPrecisionLinear.py:60-62); ap_gemm_kbit_group_pays the same for ONE ap_gemm_kbit_group
 * launch over `count` linears against calling them one by one.  The host module asks these instead of
 * keeping thresholds of its own.  Negative argument errors as for ap_gemm_kbit. */
int ap_gemm_kbit_pays(int M, int N, int K, int w_bits);
int ap_gemm_kbit_group_pays(int count, const int *N, int M, int K, int w_bits);

/* Human-readable text for a return code of the functions above. */
const char *ap_strerror(int code);

/* AP_ABI_VERSION the library was built with. */
int ap_abi_version(void);

/* Launch geometry the GEMV would use, for reports and tests: words per lane,
 * K-segments (waves) per workgroup, rows per workgroup, grid size.
 * Returns AP_OK or the same argument errors as ap_matmul_kbit. */
int ap_matmul_kbit_geometry(int M, int N, int K, int w_bits,
                            int *wpl, int *segments, int *rows, int *grid);

/* Which kernel ap_matmul_kbit would launch for one linear (output taken to be 4-byte aligned), for
 * reports and tests.  Returns AP_OK or the argument errors of ap_matmul_kbit. */
enum {
    AP_ROUTE_DOT = 0,     /* gemv_kbit_kernel: one, two or four rows per workgroup                      */
    AP_ROUTE_STREAM = 1,  /* gemvp_kbit_kernel: row pairs, 16-byte plane loads, few long waves           */
    AP_ROUTE_FINE = 2,    /* gemvf_kbit_kernel: one workgroup per row pair, 8-byte plane loads           */
    AP_ROUTE_MFMA4 = 3,   /* gemv4_kbit_kernel: 4x4x4 matrix-core kernel                                 */
    AP_ROUTE_MFMA16 = 4   /* gemm_kbit_kernel: 16x16x32 matrix-core kernel                               */
};
int ap_matmul_kbit_route(int M, int N, int K, int w_bits, int *route);
/* The same for a set of `count` linears given to ap_matmul_kbit_group: route[g] per member (all AP_ROUTE_DOT = one
 * launch for the set; anything else = a launch per member) and, if `rows` is not NULL, the weight rows per workgroup
 * the dot-product kernel would use for the set. */
int ap_matmul_kbit_group_route(int count, const int *N, int M, int K, int w_bits, int *route, int *rows);

/* Test and measurement hook, no counterpart in the reference: overrides one launch-heuristic knob
 * (which kernel variant serves a shape, grid sizes) for the whole process, so that tests can force
 * every variant onto shapes they can check and benchmarks can sweep.  Results never depend on a knob
 * beyond the 1e-2 bar of the entry points; the defaults are what measured fastest.  Names:
 * gemv_target_waves, gemv_rows, gemv_wpl, dequant_blocks_per_cu, matmul_mfma_from, gemm_split,
 * matmul_mfma4, gemv4_groups, gemm_rb2, gemv_stream, gemv_stream_waves, gemv_fine,
 * gemm_walk, gemm_walk_wgs, gemm_tiled, gemm_tile, gemm_tile_split, gemm_lookahead.  Returns AP_OK, AP_ENULL or AP_EKNOB.
 * For tests and measurements only: the knobs are plain process-wide integers, NOT thread-safe against
 * concurrent launches (a launch that races with a change sees either value); a serving process leaves
 * them alone. */
int ap_set_tuning(const char *name, int value);
int ap_get_tuning(const char *name, int *value);

/* Measurement aids, no counterpart in the reference.  ap_probe_stream only READS bytes0 bytes at buf0
 * and bytes1 bytes at buf1 (multiples of 16; buf1 may be NULL with bytes1 = 0) with 16-byte non-temporal
 * loads from `waves_per_cu` waves per CU (<= 0: 8) and writes nothing but possibly sink[0]: timed over
 * the planes and tables of a linear it is the floor any kernel over those bytes has on this machine.
 * ap_probe_write only WRITES `bytes` bytes (a multiple of 16) of `value` at dst with 16-byte non-temporal
 * stores (waves_per_cu <= 0: 32): the floor of a store-bound kernel such as ap_dequant_kbit.
 * ap_probe_empty launches one wave that does nothing: the fixed cost of a launch. */
int ap_probe_stream(const void *buf0, long long bytes0, const void *buf1, long long bytes1,
                    uint32_t *sink, int waves_per_cu, void *stream);
int ap_probe_write(void *dst, long long bytes, uint32_t value, int waves_per_cu, void *stream);
int ap_probe_empty(uint32_t *sink, void *stream);

/* ---- The rest of a decode step, for ONE new token of a Llama-architecture decoder ----------------------
 * The reference has no native code between its linears: its model wrapper hands the step to the Hugging
 * Face modules (any_precision/modules/AnyPrecisionForCausalLM.py:88-97, timed by demo.py:59-80), i.e. a
 * dozen library kernels per layer around the seven GEMVs.  These three entry points replace them in a
 * graph-captured decode step; fp16 in memory, fp32 arithmetic, one rounding per output; 16-byte aligned
 * pointers; nothing is allocated.
 *
 * ap_add_rmsnorm: for each of `rows` rows of H elements (H % 8 == 0): s = h + delta (an fp16 add; delta may
 *   be NULL), written to h_out (may alias h); x_out = s * rsqrt(mean(s^2) + eps) * weight[H]  (LlamaRMSNorm).
 * ap_silu_mul: out = gate / (1 + exp(-gate)) * up over n elements (n % 8 == 0)  (the SwiGLU gate).
 * ap_decode_attention: rotary embedding, cache append and attention of the token at cache row *pos (a device
 *   scalar, so the launch can sit in a replayed graph):
 *     qkv   [n_heads + 2 n_kv_heads, head_dim]  query, key and value heads of the token, before the rotary embedding
 *     cos_table, sin_table [max_len, head_dim / 2] fp32: cos / sin of (row * inverse frequency i)
 *     kcache, vcache [n_kv_heads, max_len, head_dim]: rows 0 .. *pos-1 are read, row *pos is written
 *     out   [n_heads * head_dim] = softmax(scale * q k^T) v per head, query head h reading key/value head
 *           h / (n_heads / n_kv_heads); rotary convention x * cos + rotate_half(x) * sin.
 *   head_dim 32, 64, 128 or 256; max_len <= 8192 (AP_ELIMIT beyond); a *pos outside 0 .. max_len-1 leaves every
 *   buffer untouched.  Calls that overlap on one cache race.
 * ap_decode_advance: the end of a greedy decode step, all on device scalars: t = argmax(logits[0 .. n)) (first index of
 *   the maximum; NaN counts as the maximum, like torch.argmax); p = *pos + 1; if p < max_len: emitted[p] = t and
 *   *pos = p; *tok = t.  One workgroup; logits 16-byte aligned. */
int ap_add_rmsnorm(const uint16_t *h, const uint16_t *delta, const uint16_t *weight, uint16_t *h_out, uint16_t *x_out,
                   int rows, int H, float eps, void *stream);
int ap_silu_mul(const uint16_t *gate, const uint16_t *up, uint16_t *out, long long n, void *stream);
int ap_decode_advance(const uint16_t *logits, int n, long long *pos, long long *tok, long long *emitted, int max_len,
                      void *stream);
int ap_decode_attention(const uint16_t *qkv, const float *cos_table, const float *sin_table, uint16_t *kcache,
                        uint16_t *vcache, const long long *pos, uint16_t *out, int n_heads, int n_kv_heads, int head_dim,
                        int max_len, float scale, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* ANYPREC_HIP_H */

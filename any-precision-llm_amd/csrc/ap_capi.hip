// C ABI of libanyprec_hip: argument checks, launch geometry, dispatch.
// The declarations and their reference counterparts are in include/anyprec_hip.h.
#include <hip/hip_runtime.h>
#include <string.h>

#include "anyprec_hip.h"
#include "ap_decode.hpp"
#include "ap_dequant.hpp"
#include "ap_gemm_launch.hpp"
#include "ap_gemmt_launch.hpp"
#include "ap_gemmw_launch.hpp"
#include "ap_gemv4_launch.hpp"
#include "ap_gemv_launch.hpp"
#include "ap_gemvf_launch.hpp"
#include "ap_gemvp_launch.hpp"
#include "ap_probe.hpp"

namespace {

using namespace ap;

// Launch-heuristic knobs.  Defaults are what measured fastest on MI355X; ap_set_tuning() overrides one for
// the whole process (tests force every kernel variant with it, benchmarks sweep with it).  Plain ints read
// at every call: a caller that changes a knob while another thread launches gets either value.
struct Knob {
    const char *name;
    int value;
};
enum {
    kGemvTargetWaves,   // waves the dot-product GEMV grid aims for (rows per workgroup follows)
    kGemvRows,          // > 0: rows per workgroup of that kernel, overrides the above
    kGemvWpl,           // > 0: words per lane of that kernel
    kDequantBlocksPerCu, // > 0: workgroups per CU the dequant grid is capped at (0: by size)
    kMatmulMfmaFrom,    // ap_matmul_kbit uses the 16x16x32 MFMA kernel from this many activation rows on
    kGemmSplit,         // > 0: K-split waves per workgroup of the fused GEMM
    kMatmulMfma4,       // 4x4x4 matrix-core kernel: 0 never, 1 where it pays, 2 for 2..8 rows wherever it fits
    kGemv4Groups,       // > 0: word groups per wave of that kernel
    kGemmRb2,           // fused GEMM, two weight-row blocks per workgroup: 0 never, 1 where it pays, 2 always
    kGemvStream,        // row-streaming GEMV: 0 never, 1 where it pays, 2 wherever it fits
    kGemvStreamWaves,   // waves per CU the row-streaming GEMV grid aims for
    kGemvFine,          // fine-grained row-pair GEMV: 0 never, 1 where it pays, 2 wherever it fits
    kGemmWalk,          // row-walking fused GEMM: 0 never, 1 where it pays, 2 wherever it fits
    kGemmWalkWgs,       // workgroups per CU its grid aims for
    kGemmTiled,         // tiled fused GEMM (ap_gemm_kbit): 0 never, 1 where it pays, 2 wherever it fits
    kGemmTile,          // > 0: blocks of 16 activation rows in its tile: 1, 2, 4 or 8
    kGemmTileSplit,     // > 0: groups of four waves per workgroup of the 64-row tile, each on its share of K: 1 or 2
    kGemmLookahead,     // K-split fused GEMM, lookups one word ahead of the matrix instructions: 0 never, 1 where it pays, 2 wherever the variant exists
    kKnobCount
};
Knob g_knobs[kKnobCount] = {
    {"gemv_target_waves", 16384}, {"gemv_rows", 0},      {"gemv_wpl", 0},     {"dequant_blocks_per_cu", 0},
    {"matmul_mfma_from", 5},      {"gemm_split", 0},     {"matmul_mfma4", 1}, {"gemv4_groups", 0},
    {"gemm_rb2", 1},              {"gemv_stream", 1},    {"gemv_stream_waves", 24},
    {"gemv_fine", 1},
    {"gemm_walk", 1},             {"gemm_walk_wgs", 1},  {"gemm_tiled", 1},   {"gemm_tile", 0},
    {"gemm_tile_split", 0},       {"gemm_lookahead", 1},
};
inline int knob(int k) { return __atomic_load_n(&g_knobs[k].value, __ATOMIC_RELAXED); }

// Compute units of the current device (256 on MI355X), looked up once per device.
int cu_count() {
    constexpr int kMaxDev = 64;
    static int cached[kMaxDev];  // 0 = not yet known
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDev) return 256;
    int n = __atomic_load_n(&cached[dev], __ATOMIC_RELAXED);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n < 1) n = 256;
        __atomic_store_n(&cached[dev], n, __ATOMIC_RELAXED);
    }
    return n;
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

int check_common(int N, int K, int w_bits) {
    if (w_bits < 3 || w_bits > 8) return AP_EBITS;
    if (N < 1 || K < 32 || (K & 31) != 0) return AP_ESHAPE;
    return AP_OK;
}

// Launch geometry for `count` linears of n[0..count) rows that share K, M and w_bits.
// Two to four activation rows on rows of at least 8192 elements (one word per lane): FOUR weight rows per workgroup,
// so that the M x 4 KB of activations a wave loads through the L1 serve four rows.  Measured against every other
// kernel on 4096 x 11008 / 14336, 5120 x 13824, 8192 x 8192, 28672 x 8192, 8192 x 28672 (two runs each):
//   M = 2: 5-13 % faster than the row-streaming and two-row kernels on rows of up to 6 waves (8192, 11008
//          elements); on longer rows mixed (-10 .. +15 %), not used;
//   M = 3, 4: 8-40 % faster than the 4x4x4 matrix-core kernel and the two-row kernel on rows of 4 waves and of
//          7 or more (8192, 13824, 14336, 28672 elements) at almost every bit-width -- the matrix-core kernel
//          needs two word groups per wave there and doubles its time from 4 bits on (5120 x 13824, M = 3, 4 bits:
//          28.9 us against 18.5) --, but 10-35 % SLOWER on rows of 11008 elements (workgroups of 6 waves: two of them
//          fit a CU at the four-row kernel's register count, three at the two-row kernel's), which keep their routes.
// Swept again after the kernels' prologues were trimmed: at M = 2 and up to 4 bits rows of 7-8 waves (13824, 14336,
// 16384 elements) are 7-13 % faster with four rows than with the row-streaming kernel that served them (4096 x 14336,
// 3 bits: 12.1 -> 10.6 us); rows of 14 waves (28672) are 22 % slower and stay with it.
bool long_rows_want_four(int M, int K, int w_bits) {
    const int W = K >> 5, S = (W + kWave - 1) / kWave;
    if (M < 2 || M > 4 || K < 8192 || S > kGemvMaxSeg) return false;
    return M == 2 ? (S <= 6 || (S <= 8 && w_bits <= 4)) : (S <= 4 || S >= 7);
}

// Four activation rows at 6-8 bits on rows of 4097..8191 elements (5120 x 5120, 13824 x 5120): four weight rows per
// workgroup too, 9-13 % faster than the 4x4x4 kernel there (equal or slower at fewer bits and at three rows).
bool mid_rows_want_four(int M, int K, int w_bits) { return M == 4 && w_bits >= 6 && K > 4096 && K < 8192; }

int gemv_geometry(int M, const int *n, int count, int K, int w_bits, GemvGeometry *geo, GemvMembers *mem) {
    long long rows = 0;
    for (int g = 0; g < count; g++) {
        const int rc = check_common(n[g], K, w_bits);
        if (rc != AP_OK) return rc;
        rows += n[g];
    }
    if (M < 1 || M > 8) return AP_EBATCH;
    const int force_wpl = knob(kGemvWpl), force_rows = knob(kGemvRows), target_waves = knob(kGemvTargetWaves);
    const int W = K >> 5;
    // One word per lane (two waves per 4096 elements of a row) measured 5-15 % faster than
    // two on planes that come from HBM, up to rows of 16384 elements; beyond (more than 8 waves
    // per row) two words per lane are 7-10 % faster (8192 x 28672), and they are needed when
    // one word per lane would take more waves than a workgroup holds.
    int wpl = 1;
    if (M <= 2 && (W & 1) == 0 && (W + kWave - 1) / kWave > 8) wpl = 2;
    if (force_wpl == 1 || (force_wpl == 2 && (W & 1) == 0 && M <= 2)) wpl = force_wpl;
    const int seg = kWave * wpl;
    const int S = (W + seg - 1) / seg;
    if (S > kGemvMaxSeg) return AP_ELIMIT;
    // One row per workgroup until that would launch more than target_waves waves, then two
    // (the second row reuses the activation registers; more rows lengthen the compute
    // tail).  From M = 3 on the activations are the larger load: at least two rows (four in the cases below).
    // At 3-4 bits (least work per wave) and for a single linear at two activation rows the switch comes at three quarters of that:
    // 5120 x 5120 (15360 waves) is 8-15 % faster with two rows there (M = 1: within 3 % either way from 5 bits
    // on); 4096 x 4096 (8192 waves) keeps one.
    const long long tw = target_waves > 0 ? ((w_bits <= 4 || (M == 2 && count == 1)) ? (long long)target_waves * 3 / 4 : target_waves) : 1;
    int R = force_rows > 0 ? force_rows : (rows * S >= tw ? 2 : 1);
    // Two activation rows at up to 4 bits: two weight rows from 4096 waves on (4096 x 4096, 8192 waves: 7-9 % faster,
    // 3 bits 5.5 -> 5.0 us; 1024 x 4096, 2048 waves, is 6 % slower with two and keeps one; from 5 bits on 4096 x 4096
    // is 3-11 % slower with two).
    if (force_rows <= 0 && M == 2 && count == 1 && w_bits <= 4 && rows * S >= 4096) R = 2;
    R = (R >= 2 || M > 2) ? 2 : 1;
    // Four rows per workgroup (one activation row, one word per lane): the activations a wave holds then serve
    // four rows, which halves their traffic through the L1 once more, at the price of half the waves.  Measured
    // 3-6 % faster (two boxes, run-to-run noise about as large) on single linears of at least 28000 waves at up to
    // 4 bits (14336 x 4096, 4096 x 14336) and, with rows of at least 8192 elements, at every bit-width
    // (8192 x 8192, 28672 x 8192); equal or slower on the Llama-2-7B shapes, so those keep two.
    // Launches of several linears at 2..4 activation rows (q/k/v, gate/up of the 7B / 8B / 13B / 70B models, swept at
    // 3, 4, 5, 8 bits): four rows at M = 3, 4 at every bit-width (the one launch is 20-46 % faster than a 4x4x4
    // launch per member and 5-20 % faster than two rows), and at M = 2 at up to 4 bits (4-12 %; 3-9 % slower at 5 bits).
    // At the highest bit-widths the lookups want more waves in flight: ONE row per workgroup up to 32768 waves is
    // 8-15 % faster at 7-8 bits for launches of several linears (q/k/v: 3 x 4096 x 4096 = 24576 waves) and 2-7 %
    // faster at 8 bits for single wide ones of short rows (11008 / 14336 x 4096).  At 3-4 bits launches of several
    // linears are 3-6 % faster with FOUR rows from 20000 waves on.
    if (M == 1 && wpl == 1 && force_rows <= 0 && rows * S <= 32768 &&
        (count > 1 ? w_bits >= 7 : (w_bits == 8 && K < 8192)))
        R = 1;
    if (M <= 4 && wpl == 1) {
        const long long waves = rows * S;
        const bool pays = M == 1 ? (count == 1 ? waves >= 28000 && (w_bits <= 4 || (K >= 8192 && waves >= 32768))
                                               : waves >= 20000 && w_bits <= 4)
                                 : long_rows_want_four(M, K, w_bits) || mid_rows_want_four(M, K, w_bits) ||
                                   (count > 1 && (M >= 3 || w_bits <= 4));
        if (force_rows == 4 || (force_rows <= 0 && pays)) R = 4;
    }
    geo->wpl = wpl;
    geo->S = S;
    geo->R = R;
    long long grid = 0;
    for (int g = 0; g < count; g++) {
        grid += (n[g] + R - 1) / R;
        if (mem) {
            mem->n[g] = n[g];
            mem->wg_end[g] = (int)grid;
        }
    }
    if (grid > 0x7fffffffLL) return AP_ELIMIT;
    geo->grid = (int)grid;
    if (mem) mem->count = count;
    return AP_OK;
}

// One launch of the dequantiser over `count` linears (arguments already checked): fills the member table and sizes the grid.
template <int BITS>
void launch_dequant(const DequantMembers &mem, hipStream_t stream) {
    const long long items = mem.items;  // 64-word segments of all members
    long long blocks = (items + kDequantWaves - 1) / kDequantWaves;
    // One item per wave (the hardware hands out workgroups as others retire) measured best or within 1-2 % of best
    // from 15 workgroups per CU on, against caps of 3..64 per CU with waves striding over the rest (the seven linears of
    // a Llama-2-7B layer in one launch: 85.5 / 107.5 us at 3 / 8 bits against 90 / 110 at 64 per CU).  A launch of 5..12
    // workgroups per CU is resident all at once -- one burst of reads, then one of writes: capped at 5 per CU its
    // waves take one or two items each, the second item's loads fly while the first one's stores drain, and it is 4-6 %
    // faster (4096 x 4096: 9.3 -> 8.8 us at 3 bits, 12.4 -> 11.6 at 8).  The knob overrides when positive.
    const long long cus = cu_count();
    long long cap = blocks;
    if (knob(kDequantBlocksPerCu) > 0) cap = cus * knob(kDequantBlocksPerCu);
    else if (blocks > 5 * cus && blocks <= 12 * cus) cap = 5 * cus;
    if (blocks > cap) blocks = cap;
    dequant_kbit_kernel<BITS><<<dim3((unsigned)blocks), dim3(kDequantWaves * kWave), 0, stream>>>(mem);
}

// hipGetLastError() returns AND clears the thread's sticky error, whoever left it: an entry point
// drains it before its first launch, so that launch_status() reports only what its own launches did.
void drain_stale_error() { (void)hipGetLastError(); }

int launch_status() {
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? AP_OK : (int)e;
}

}  // namespace

extern "C" {

int ap_abi_version(void) { return AP_ABI_VERSION; }

const char *ap_strerror(int code) {
    switch (code) {
        case AP_OK: return "ok";
        case AP_ENULL: return "null pointer argument";
        case AP_EBITS: return "w_bits must be in 3..8";
        case AP_ESHAPE: return "need N >= 1 and K a positive multiple of 32";
        case AP_EALIGN: return "pointer not 16-byte aligned";
        case AP_EBATCH: return "batch M outside the range this entry point serves";
        case AP_ELIMIT: return "size exceeds the launch geometry limits";
        case AP_EKNOB: return "unknown tuning knob";
        default: break;
    }
    if (code > 0) return hipGetErrorString((hipError_t)code);
    return "unknown error code";
}

int ap_set_tuning(const char *name, int value) {
    if (!name) return AP_ENULL;
    for (int k = 0; k < kKnobCount; k++)
        if (strcmp(name, g_knobs[k].name) == 0) {
            __atomic_store_n(&g_knobs[k].value, value, __ATOMIC_RELAXED);
            return AP_OK;
        }
    return AP_EKNOB;
}

int ap_get_tuning(const char *name, int *value) {
    if (!name || !value) return AP_ENULL;
    for (int k = 0; k < kKnobCount; k++)
        if (strcmp(name, g_knobs[k].name) == 0) {
            *value = knob(k);
            return AP_OK;
        }
    return AP_EKNOB;
}

int ap_probe_stream(const void *buf0, long long bytes0, const void *buf1, long long bytes1, uint32_t *sink,
                    int waves_per_cu, void *stream) {
    if (!buf0 || !sink || (bytes1 > 0 && !buf1)) return AP_ENULL;
    if (bytes0 < 0 || bytes1 < 0 || (bytes0 & 15) || (bytes1 & 15)) return AP_ESHAPE;
    if (!aligned16(buf0) || (bytes1 > 0 && !aligned16(buf1))) return AP_EALIGN;
    if (waves_per_cu < 1) waves_per_cu = 8;
    const long long units = (bytes0 + bytes1) >> 4;
    long long blocks = (long long)cu_count() * waves_per_cu / kProbeWaves;
    const long long need = (units + kProbeWaves * kWave - 1) / (kProbeWaves * kWave);
    if (blocks > need) blocks = need;
    if (blocks < 1) blocks = 1;
    drain_stale_error();
    probe_stream_kernel<<<dim3((unsigned)blocks), dim3(kProbeWaves * kWave), 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<const u32x4 *>(buf0), bytes0 >> 4, static_cast<const u32x4 *>(buf1), bytes1 >> 4, sink);
    return launch_status();
}

int ap_probe_write(void *dst, long long bytes, uint32_t value, int waves_per_cu, void *stream) {
    if (!dst) return AP_ENULL;
    if (bytes < 0 || (bytes & 15)) return AP_ESHAPE;
    if (!aligned16(dst)) return AP_EALIGN;
    if (waves_per_cu < 1) waves_per_cu = 32;
    const long long units = bytes >> 4;
    long long blocks = (long long)cu_count() * waves_per_cu / kProbeWaves;
    const long long need = (units + kProbeWaves * kWave - 1) / (kProbeWaves * kWave);
    if (blocks > need) blocks = need;
    if (blocks < 1) blocks = 1;
    drain_stale_error();
    probe_write_kernel<<<dim3((unsigned)blocks), dim3(kProbeWaves * kWave), 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<u32x4 *>(dst), units, value);
    return launch_status();
}

int ap_probe_empty(uint32_t *sink, void *stream) {
    if (!sink) return AP_ENULL;
    drain_stale_error();
    probe_empty_kernel<<<dim3(1), dim3(kWave), 0, static_cast<hipStream_t>(stream)>>>(sink);
    return launch_status();
}

int ap_add_rmsnorm(const uint16_t *h, const uint16_t *delta, const uint16_t *weight, uint16_t *h_out, uint16_t *x_out,
                   int rows, int H, float eps, void *stream) {
    if (!h || !weight || !h_out || !x_out) return AP_ENULL;
    if (rows < 1 || H < 8 || (H & 7)) return AP_ESHAPE;
    if (!aligned16(h) || !aligned16(weight) || !aligned16(h_out) || !aligned16(x_out) || (delta && !aligned16(delta)))
        return AP_EALIGN;
    drain_stale_error();
    add_rmsnorm_kernel<<<dim3(rows), dim3(kNormThreads), 0, static_cast<hipStream_t>(stream)>>>(
        reinterpret_cast<const half_t *>(h), reinterpret_cast<const half_t *>(delta), reinterpret_cast<const half_t *>(weight),
        reinterpret_cast<half_t *>(h_out), reinterpret_cast<half_t *>(x_out), H, eps);
    return launch_status();
}

int ap_silu_mul(const uint16_t *gate, const uint16_t *up, uint16_t *out, long long n, void *stream) {
    if (!gate || !up || !out) return AP_ENULL;
    if (n < 8 || (n & 7)) return AP_ESHAPE;
    if (!aligned16(gate) || !aligned16(up) || !aligned16(out)) return AP_EALIGN;
    const long long blocks = (n / 8 + 255) / 256;
    drain_stale_error();
    silu_mul_kernel<<<dim3((unsigned)(blocks < 4096 ? blocks : 4096)), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(
        reinterpret_cast<const half_t *>(gate), reinterpret_cast<const half_t *>(up), reinterpret_cast<half_t *>(out), n);
    return launch_status();
}

int ap_decode_advance(const uint16_t *logits, int n, long long *pos, long long *tok, long long *emitted, int max_len,
                      void *stream) {
    if (!logits || !pos || !tok || !emitted) return AP_ENULL;
    if (n < 1 || max_len < 1) return AP_ESHAPE;
    if (!aligned16(logits)) return AP_EALIGN;
    drain_stale_error();
    decode_advance_kernel<<<dim3(1), dim3(kAdvanceThreads), 0, static_cast<hipStream_t>(stream)>>>(
        reinterpret_cast<const half_t *>(logits), n, pos, tok, emitted, max_len);
    return launch_status();
}

int ap_decode_attention(const uint16_t *qkv, const float *cos_table, const float *sin_table, uint16_t *kcache,
                        uint16_t *vcache, const long long *pos, uint16_t *out, int n_heads, int n_kv_heads, int head_dim,
                        int max_len, float scale, void *stream) {
    if (!qkv || !cos_table || !sin_table || !kcache || !vcache || !pos || !out) return AP_ENULL;
    if (n_heads < 1 || n_kv_heads < 1 || n_heads % n_kv_heads) return AP_ESHAPE;
    if (head_dim != 32 && head_dim != 64 && head_dim != 128 && head_dim != 256) return AP_ESHAPE;
    if (max_len < 1 || max_len > kAttnMaxLen) return AP_ELIMIT;
    if (!aligned16(qkv) || !aligned16(kcache) || !aligned16(vcache) || !aligned16(out)) return AP_EALIGN;
    const half_t *q = reinterpret_cast<const half_t *>(qkv);
    half_t *kc = reinterpret_cast<half_t *>(kcache), *vc = reinterpret_cast<half_t *>(vcache), *o = reinterpret_cast<half_t *>(out);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const dim3 grid(n_heads), block(kAttnThreads);
    drain_stale_error();
    switch (head_dim) {
        case 32: decode_attention_kernel<32><<<grid, block, 0, st>>>(q, cos_table, sin_table, kc, vc, pos, o, n_heads, n_kv_heads, max_len, scale); break;
        case 64: decode_attention_kernel<64><<<grid, block, 0, st>>>(q, cos_table, sin_table, kc, vc, pos, o, n_heads, n_kv_heads, max_len, scale); break;
        case 128: decode_attention_kernel<128><<<grid, block, 0, st>>>(q, cos_table, sin_table, kc, vc, pos, o, n_heads, n_kv_heads, max_len, scale); break;
        default: decode_attention_kernel<256><<<grid, block, 0, st>>>(q, cos_table, sin_table, kc, vc, pos, o, n_heads, n_kv_heads, max_len, scale); break;
    }
    return launch_status();
}

int ap_dequant_kbit(const uint32_t *qweight, const uint16_t *lut, uint16_t *out, int N, int K, int w_bits,
                    void *stream) {
    return ap_dequant_kbit_group(1, &qweight, &lut, &out, &N, &K, w_bits, stream);
}

int ap_dequant_kbit_group(int count, const uint32_t *const *qweight, const uint16_t *const *lut, uint16_t *const *out,
                          const int *N, const int *K, int w_bits, void *stream) {
    if (!qweight || !lut || !out || !N || !K) return AP_ENULL;
    if (count < 1 || count > kDequantMaxGroup) return AP_ELIMIT;
    DequantMembers mem = {};
    long long items = 0;
    for (int g = 0; g < count; g++) {
        if (!qweight[g] || !lut[g] || !out[g]) return AP_ENULL;
        const int rc = check_common(N[g], K[g], w_bits);
        if (rc != AP_OK) return rc;
        if (!aligned16(qweight[g]) || !aligned16(lut[g]) || !aligned16(out[g])) return AP_EALIGN;
        const long long segs = (long long)N[g] * (((K[g] >> 5) + kWave - 1) / kWave);
        items += segs;
        if (items > 0x7fffffffLL) return AP_ELIMIT;  // the kernel numbers the segments of a launch in 32 bits
        mem.seg_magic[g] = reciprocal_floor((uint32_t)(((K[g] >> 5) + kWave - 1) / kWave));
        mem.qweight[g] = qweight[g];
        mem.lut[g] = lut[g];
        mem.out[g] = out[g];
        mem.N[g] = N[g];
        mem.K[g] = K[g];
        mem.item_end[g] = (int)items;
    }
    mem.items = (int)items;
    mem.count = count;
    hipStream_t st = static_cast<hipStream_t>(stream);
    drain_stale_error();
    switch (w_bits) {
        case 3: launch_dequant<3>(mem, st); break;
        case 4: launch_dequant<4>(mem, st); break;
        case 5: launch_dequant<5>(mem, st); break;
        case 6: launch_dequant<6>(mem, st); break;
        case 7: launch_dequant<7>(mem, st); break;
        default: launch_dequant<8>(mem, st); break;
    }
    return launch_status();
}

int ap_matmul_kbit_geometry(int M, int N, int K, int w_bits, int *wpl, int *segments, int *rows, int *grid) {
    GemvGeometry geo;
    const int rc = gemv_geometry(M, &N, 1, K, w_bits, &geo, nullptr);
    if (rc != AP_OK) return rc;
    if (wpl) *wpl = geo.wpl;
    if (segments) *segments = geo.S;
    if (rows) *rows = geo.R;
    if (grid) *grid = geo.grid;
    return AP_OK;
}

}  // extern "C"

namespace {

// The row-walking fused GEMM serves up to 32 activation rows on rows of a multiple of 128 elements that its
// K-split waves cover with one step of 512 elements each (two steps at up to 16 activation rows and 5 bits:
// beyond, the double-buffered planes no longer fit the registers).
bool gemmw_geometry(int M, int N, int K, int w_bits, GemmwGeometry *geo) {
    const int W = K >> 5;
    if (M < 1 || M > kGemmwMaxM || (W & 3) != 0 || N < 16) return false;
    const int steps = (W + 15) / 16;
    const int mb = (M + 15) / 16, spw = steps <= kGemmMaxSplit ? 1 : 2;
    if (steps > 2 * kGemmMaxSplit || mb * spw > 2 || (spw == 2 && w_bits > 5)) return false;
    const int ks = (steps + spw - 1) / spw;
    if (ks < 4) return false;
    if ((long long)M * K * 2 > 0xffffffffLL) return false;
    const int nblocks = (N + 15) / 16;
    int per_cu = knob(kGemmWalkWgs);
    if (per_cu < 1) per_cu = 1;
    const long long wgs = (long long)cu_count() * per_cu;
    const long long rounds = (nblocks + wgs - 1) / wgs;
    geo->mb = mb;
    geo->spw = spw;
    geo->ks = ks;
    geo->grid = (int)((nblocks + rounds - 1) / rounds);  // every workgroup walks `rounds` blocks (the last ones one fewer)
    return true;
}

// Tile of the tiled fused GEMM (ap_gemmt.hpp) for a shape; false if the kernel does not serve it.  64 weight rows x
// 64 activation rows unless that makes several workgroups per CU: then 64 x 128, which halves the table lookups per
// matrix instruction (measured on 4096 x 4096, 11008 / 14336 x 4096, 4096 x 11008, 5120 x 5120, 8192 x 8192 at 48..512
// rows: the larger tile wins from about 3 workgroups of the smaller one per CU on at 3 bits, from 1.3 on at 4+ bits).
// Grids of at most one small tile per CU run it with two groups of waves, each on half of K (4096 x 4096 at 128..256
// rows: 38 us against 50 at 8 bits, 26 against 37 at 4 bits, where this form also has room for the pair table; 4096 x
// 11008: 65 against 100 at 4 bits); with more tiles than
// CUs the second group only takes LDS from the next workgroup (11008 x 4096, 256 rows, 3 bits: 71 us against 56).
bool gemmt_geometry(int M, long long tiles_n, int K, int w_bits, GemmtGeometry *geo) {
    if ((K & 127) != 0 || (long long)M * K * 2 > 0xffffffffLL || tiles_n > 0x7fffffffLL) return false;
    const int forced = knob(kGemmTile), force_kh = knob(kGemmTileSplit);
    const long long small = tiles_n * ((M + 63) / 64);  // tiles of 64 x 64
    int mbw = 4;
    if (forced > 0) {
        if (forced != 1 && forced != 2 && forced != 4 && forced != 8) return false;
        if (forced < 4 && K < 1024) return false;  // tiles of 16 and 32 rows exist in the two-half form only
        mbw = forced;
    } else if (M > 64) {
        // Tiles of 128 activation rows once the 64-row tiles no longer fit the CUs in one round of the two-half form --
        // from 5 bits on as soon as they exceed the CUs (5120 x 5120 at 256 rows, 320 tiles: 47 / 49 / 56 us at 5 / 6 / 8
        // bits against 52 / 56 / 73 with one group of waves per 64-row tile); at 4 bits, whose two-half form has the
        // pair table, from 1.5 tiles per CU (up to there two rounds of that form: 44 us against 47); at 3 bits from 3
        // tiles per CU (one group of waves per 64-row tile is as fast up to there).
        const long long cus = cu_count();
        if (w_bits == 3 ? small >= 3 * cus : (w_bits == 4 ? 2 * small > 3 * cus : small > cus)) mbw = 8;
    }
    // A grid that leaves CUs idle takes the narrowest tile that still gives no CU a second workgroup: more workgroups
    // dequantise the same weights, each for fewer activation rows (4096 x 4096 at 64 rows, 3 bits: 14 us with four
    // times 64 tiles of 16 rows against 19 with 64 tiles of 64; at 128 rows 16 us with tiles of 32 against 19).
    if (forced <= 0 && force_kh != 1 && mbw == 4 && K >= 1024) {
        if (tiles_n * ((M + 15) / 16) <= cu_count()) mbw = 1;
        else if (tiles_n * ((M + 31) / 32) <= cu_count()) mbw = 2;
    }
    geo->mbw = mbw;
    // two K halves need at least two steps of 512 elements
    const bool halves = small <= cu_count() || (w_bits == 4 && 2 * small <= 3 * (long long)cu_count());
    geo->kh = mbw < 4 || (mbw == 4 && K >= 1024 && (force_kh == 2 || (force_kh <= 0 && halves))) ? 2 : 1;
    geo->grid_n = (int)tiles_n;  // tiles of 64 weight rows (of all linears of the launch)
    geo->grid_m = (M + 16 * mbw - 1) / (16 * mbw);
    return (tiles_n + 7) / 8 * 8 * (long long)geo->grid_m <= 0x7fffffffLL;  // a one-dimensional grid, padded to groups of 8
}

// Where the tiled kernel is the fastest fused form (same sweep, and the linear shapes of the 7B / 8B / 13B / 70B layers
// at 16..256 rows, against the K-split kernel, which serves more than 128 rows in chunks of 128).  Its time grows with
// the activation rows in steps of a tile (16, 32 or 64 rows, gemmt_geometry), while the K-split kernel's grows with
// every block of 16 rows and steps up beyond 32 (4096 x 4096 at 128 rows: 15 / 19 / 22 / 29 us at 3 / 4 / 5 / 8 bits
// against 34-36; rows of more than 4096 elements at 8 bits: 1.8-2x, e.g. 13824 x 5120 83 us against 171).  Wide linears
// -- at least 8192 rows of at most 4096 elements, or more than 10240 rows of any length -- take it from 17 rows on
// (11008 x 4096 at 48 rows: 20-36 us against 33-48; 14336 x 4096 at 32 rows: 18-33 against 22-36); those of at most
// 16384 rows, whose grid has room for tiles of 16 activation rows, from 9 up to 4 bits or on rows of more than 4096
// elements (11008 x 4096 at 16 rows, 3 bits: 12.8 us against 14.3; 13824 x 5120: 17-37 against 20-45; 28672 x 8192
// at 16 rows would be 59-90 against 45-75).  Linears of 5120..10240 rows of more than 4096 elements from 33 rows on (5120 x 5120 at 48 rows:
// 18-36 us against 28-41), from 17 at 3 bits (8192 x 8192 at 32 rows: 19.7 against 21.9); the rest (up to 4096 rows)
// from 33 rows on at 3 and 4 bits (4096 x 4096 at 64 rows: 13-15 us against 19), from 49 at 5 bits (4096 x 11008 at 64
// rows: 45 against 50), 65 at 6, 81 at 7 and 8 (4096 x 11008 at 96 rows, 8 bits: 68 against 75).
bool gemmt_pays(int M, int N, int K, int w_bits) {
    if ((N >= 8192 && K <= 4096) || N > 10240) return M > 16 || (M > 8 && N <= 16384 && (w_bits <= 4 || K > 4096));
    if (N >= 5120 && K > 4096) return M > 32 || (M > 16 && w_bits == 3);
    return M > (w_bits <= 4 ? 32 : (w_bits == 5 ? 48 : (w_bits == 6 ? 64 : 80)));
}

// Launch of the fused dequant -> MFMA kernel (arguments already checked).
int run_gemm(const uint16_t *x, const uint32_t *qweight, const uint16_t *lut, uint16_t *out, int M, int N, int K,
             int w_bits, hipStream_t st) {
    // the kernels address the activations, and a row inside a plane, with 32-bit byte offsets
    if ((long long)M * K * 2 > 0xffffffffLL || (long long)N * (K >> 5) * 4 > 0xffffffffLL) return AP_ELIMIT;
    {
        GemmwGeometry wgeo;
        const int mode = knob(kGemmWalk);
        // Where it pays (measured on 11008 / 14336 x 4096 and 28672 x 8192; 5-18 %): linears with at least 2.5
        // blocks of rows per CU to walk, at 17..32 activation rows or at 8 bits with one step per wave, and from 9
        // rows on with two (from 5 rows at up to 4 bits: 6-21 % on 28672 x 8192).  Elsewhere the one-shot kernels are as fast or faster (fewer rows: nothing to walk; fewer
        // activation rows at low bit-widths: their short waves hide the lookup latency better).
        // With two steps per wave it needs twice the rows (28672 x 8192: 5-21 %; on 13824 x 5120 the two-block
        // one-shot kernel is up to 20 % faster).
        const bool pays = gemmw_geometry(M, N, K, w_bits, &wgeo) && N >= 40 * wgeo.spw * cu_count() &&
                          (wgeo.spw == 1 ? (M > 16 || w_bits == 8) : (M > 8 || (M >= 5 && w_bits <= 4)));
        if (mode > 0 && (mode >= 2 ? gemmw_geometry(M, N, K, w_bits, &wgeo) : pays)) {
            switch (w_bits) {
                case 3: launch_gemmw<3>(wgeo, x, qweight, lut, out, M, N, K, st); break;
                case 4: launch_gemmw<4>(wgeo, x, qweight, lut, out, M, N, K, st); break;
                case 5: launch_gemmw<5>(wgeo, x, qweight, lut, out, M, N, K, st); break;
                case 6: launch_gemmw<6>(wgeo, x, qweight, lut, out, M, N, K, st); break;
                case 7: launch_gemmw<7>(wgeo, x, qweight, lut, out, M, N, K, st); break;
                default: launch_gemmw<8>(wgeo, x, qweight, lut, out, M, N, K, st); break;
            }
            return launch_status();
        }
    }
    GemmGeometry geo;
    geo.mb = (M + 15) / 16;
    const int W = K >> 5;
    // Two blocks of 16 weight rows per workgroup halve the L2 traffic of the activations, which
    // bounds this kernel, but also the number of workgroups, and they need twice the plane
    // registers: measured faster from 9 activation rows on, on linears of at least 8192 rows -- at
    // 3 bits, and at up to 5 bits (6 with two activation row blocks) when the linear has at least
    // 56 M weights (14336 x 4096, 8192 x 8192, 28672 x 8192: 5-25 %).
    const int rb_mode = knob(kGemmRb2);  // 0 never, 1 where it pays, 2 wherever the kernel allows
    const bool rb_fits = (W & 3) == 0 && N >= 32;
    // Linears of 5120..8191 rows (5120 x 5120, 5120 x 13824; swept later) gain as much: 19-38 % at 3 bits, 3-22 % at
    // 5 bits; and at 8 bits up to 16 activation rows gain 8-16 % wherever a wave has more than one step (rows of
    // more than 4096 elements: 5120 x 5120, 13824 x 5120, 5120 x 13824, 8192 x 8192, 8192 x 28672).
    const bool big = (long long)N * K >= 56LL << 20;
    const bool low_bits = w_bits <= 4 || (w_bits <= (geo.mb >= 2 ? 6 : 5) && (big || N < 8192));  // 4 bits: 11008 x 4096, 7-10 %
    const bool rb_pays = N >= 5120 && (M > 8 ? (low_bits || (w_bits == 8 && M <= 16 && K > 4096))
                                             : (M >= 5 && ((w_bits == 3 && big && N >= 8192) ||  // 14336 x 4096 at 5..8 rows: 6-18 %
                                                           (K >= 8192 && N <= 8192))));  // 5120 x 13824, 8192 x 28672, 8192 x 8192: 5-17 %
    geo.rb = (rb_fits && (rb_mode >= 2 || (rb_mode == 1 && rb_pays))) ? 2 : 1;
    if (geo.rb == 2 && geo.mb > 2) {
        // the two-block variant exists for up to 32 activation rows: more go in chunks of 32 (the
        // planes are re-read per chunk, which still costs less than one launch of the one-block variant)
        for (int m0 = 0; m0 < M; m0 += 32) {
            const int r = run_gemm(x + (size_t)m0 * K, qweight, lut, out + (size_t)m0 * N, M - m0 < 32 ? M - m0 : 32, N, K,
                                   w_bits, st);
            if (r != AP_OK) return r;
        }
        return AP_OK;
    }
    geo.grid = (N + 16 * geo.rb - 1) / (16 * geo.rb);
    const int steps = (W & 3) == 0 ? (W + 15) / 16 : (W + 3) / 4;  // the kernel's steps along K
    // As many K-split waves as a workgroup holds: every split measured slower with fewer
    // (the grid alone, N/16 workgroups, is far too small to fill 256 CUs).
    int ks = knob(kGemmSplit) > 0 ? knob(kGemmSplit) : kGemmMaxSplit;
    if (ks > kGemmMaxSplit) ks = kGemmMaxSplit;
    if (ks > steps) ks = steps;
    if (ks < 1) ks = 1;
    geo.ks = ks;
    // Lookups one word ahead of the matrix instructions where a CU holds one workgroup and nothing else covers a
    // wave's waits for its lookups (4096-row linears: 2-7 %); with several workgroups per CU the same variant is 5-20 %
    // slower, and at 8 bits with one step per wave and one block of activation rows 3-4 % (4096 x 4096).
    const int la_mode = knob(kGemmLookahead);
    const bool la_fits = geo.rb == 1 && geo.mb <= 2 && (W & 3) == 0;
    const bool la_pays = geo.grid <= cu_count() && !(w_bits == 8 && geo.mb == 1 && steps <= ks);
    geo.lookahead = la_fits && (la_mode >= 2 || (la_mode == 1 && la_pays)) ? 1 : 0;
    switch (w_bits) {
        case 3: launch_gemm<3>(geo, x, qweight, lut, out, M, N, K, st); break;
        case 4: launch_gemm<4>(geo, x, qweight, lut, out, M, N, K, st); break;
        case 5: launch_gemm<5>(geo, x, qweight, lut, out, M, N, K, st); break;
        case 6: launch_gemm<6>(geo, x, qweight, lut, out, M, N, K, st); break;
        case 7: launch_gemm<7>(geo, x, qweight, lut, out, M, N, K, st); break;
        default: launch_gemm<8>(geo, x, qweight, lut, out, M, N, K, st); break;
    }
    return launch_status();
}

// The row-streaming GEMV serves rows of a multiple of 128 elements (16-byte plane loads), an even number
// of rows (it walks row pairs and stores them as one dword) and up to 4 activation rows.
bool gemvp_fits(const uint16_t *out, int M, int N, int K) {
    const int W = K >> 5;
    return M >= 1 && M <= kGemvpMaxM && (W & 3) == 0 && (N & 1) == 0 &&
           (W + 127) / 128 <= kGemvpMaxSeg && (reinterpret_cast<uintptr_t>(out) & 3u) == 0;
}

int run_gemvp(const uint16_t *x, const uint32_t *qweight, const uint16_t *lut, uint16_t *out, int M, int N, int K,
              int w_bits, hipStream_t st) {
    GemvpGeometry geo;
    const int W = K >> 5, pairs = N >> 1;
    geo.S = (W + 127) / 128;
    // As many workgroups as keep `gemv_stream_waves` waves on every CU, each walking the same number
    // of row pairs (+-1): a grid a little smaller than the cap beats a ragged last round.
    int wpc = knob(kGemvStreamWaves);
    if (wpc < 1) wpc = 1;
    long long cap = (long long)cu_count() * wpc / geo.S;
    if (cap < 1) cap = 1;
    const long long rounds = (pairs + cap - 1) / cap;
    geo.grid = (int)((pairs + rounds - 1) / rounds);
    switch (w_bits) {
        case 3: launch_gemvp<3>(M, geo, x, qweight, lut, out, N, K, st); break;
        case 4: launch_gemvp<4>(M, geo, x, qweight, lut, out, N, K, st); break;
        case 5: launch_gemvp<5>(M, geo, x, qweight, lut, out, N, K, st); break;
        case 6: launch_gemvp<6>(M, geo, x, qweight, lut, out, N, K, st); break;
        case 7: launch_gemvp<7>(M, geo, x, qweight, lut, out, N, K, st); break;
        default: launch_gemvp<8>(M, geo, x, qweight, lut, out, N, K, st); break;
    }
    return launch_status();
}

// The fine-grained row-pair GEMV serves rows of a multiple of 64 elements (8-byte plane loads), an even
// number of rows and up to 4 activation rows.
bool gemvf_fits(const uint16_t *out, int M, int N, int K) {  // out == nullptr: taken to be aligned
    const int W = K >> 5;
    return M >= 1 && M <= kGemvfMaxM && (W & 1) == 0 && (N & 1) == 0 &&
           (W + 63) / 64 <= kGemvfMaxSeg && (reinterpret_cast<uintptr_t>(out) & 3u) == 0;
}

int run_gemvf(const uint16_t *x, const uint32_t *qweight, const uint16_t *lut, uint16_t *out, int M, int N, int K,
              int w_bits, hipStream_t st) {
    GemvfGeometry geo;
    geo.S = ((K >> 5) + 63) / 64;
    geo.grid = N >> 1;
    switch (w_bits) {
        case 3: launch_gemvf<3>(M, geo, x, qweight, lut, out, N, K, st); break;
        case 4: launch_gemvf<4>(M, geo, x, qweight, lut, out, N, K, st); break;
        case 5: launch_gemvf<5>(M, geo, x, qweight, lut, out, N, K, st); break;
        case 6: launch_gemvf<6>(M, geo, x, qweight, lut, out, N, K, st); break;
        case 7: launch_gemvf<7>(M, geo, x, qweight, lut, out, N, K, st); break;
        default: launch_gemvf<8>(M, geo, x, qweight, lut, out, N, K, st); break;
    }
    return launch_status();
}

int run_gemv4(const uint16_t *x, const uint32_t *qweight, const uint16_t *lut, uint16_t *out, int M, int N, int K,
              int w_bits, hipStream_t st) {
    Gemv4Geometry geo;
    if (M > 8) return AP_EBATCH;
    const int W = K >> 5;
    if ((long long)N * W * 4 > 0xffffffffLL) return AP_ELIMIT;  // the kernel addresses a row inside a plane with 32 bits
    if (M > 4) {
        // two groups of four activation rows: four row quads per workgroup, one word group per wave
        geo.mg = 2;
        geo.rq = 4;
        geo.G = 1;
        geo.S = (W + 15) / 16;
        if (geo.S > kGemv4MaxSegTwo) return AP_ELIMIT;
    } else {
        geo.mg = 1;
        geo.rq = 2;
        // one word group per wave (with two row quads: 64 weights per lane, as in the dot-product kernel)
        // unless the row is so long that a workgroup could not hold its waves
        int G = knob(kGemv4Groups) > 0 ? knob(kGemv4Groups) : 1;
        if (G != 1 && G != 2 && G != 4) G = 1;
        while (G < 4 && (W + 16 * G - 1) / (16 * G) > kGemv4MaxSeg) G *= 2;
        geo.G = G;
        geo.S = (W + 16 * G - 1) / (16 * G);
        if (geo.S > kGemv4MaxSeg) return AP_ELIMIT;
    }
    geo.grid = (N + 4 * geo.rq - 1) / (4 * geo.rq);
    switch (w_bits) {
        case 3: launch_gemv4<3>(geo, x, qweight, lut, out, M, N, K, st); break;
        case 4: launch_gemv4<4>(geo, x, qweight, lut, out, M, N, K, st); break;
        case 5: launch_gemv4<5>(geo, x, qweight, lut, out, M, N, K, st); break;
        case 6: launch_gemv4<6>(geo, x, qweight, lut, out, M, N, K, st); break;
        case 7: launch_gemv4<7>(geo, x, qweight, lut, out, M, N, K, st); break;
        default: launch_gemv4<8>(geo, x, qweight, lut, out, M, N, K, st); break;
    }
    return launch_status();
}

// ---------------------------------------------------------------------------------------------------------------
// Routing: which kernel serves each of `count` linears that share x, M, K and w_bits.
//
// Every rule below is a threshold fitted to measurements on the linears of the Llama-2-7B / Llama-3-8B / 13B / 70B
// decoder layers (and their q/k/v and gate/up sets), cold weights, two runs each; `bench.py --workload
// routing_audit` re-measures the default choice against every alternative.  Three parts:
//   forced_route     a kernel forced by a tuning knob (tests, sweeps);
//   few_rows_route   M below the knob matmul_mfma_from (1..4 by default): the dot-product family and the 4x4x4 kernel;
//   many_rows_route  M from that knob on (5..8): the matrix-core kernels, and the dot-product kernel where it still wins.
// The dot-product kernels other than gemv_kbit_kernel serve one linear per launch and stay within +-6 % of it on every
// shape -- a launch is bound by its latency chain (dispatch, first loads, table staging, last compute, segment sums)
// and by what the memory system delivers to a burst of requests, not by the instruction count -- so they are used
// only where they won by 3 % or more.

struct RouteQuery {
    int M, count, K, w_bits;
    const int *N;
    int lo, hi;        // fewest / most rows of a member
    long long rows;    // all members together
    bool fits_fine, fits_stream;  // every member can run that kernel
    const GemvGeometry *geo;                    // of the joint dot-product launch
};

bool single(const RouteQuery &q) { return q.count == 1; }

// The 4x4x4 kernel's own limits (word groups per wave, waves per workgroup).
bool mfma4_fits(const RouteQuery &q) {
    const int W = q.K >> 5;
    if (q.M < 2 || q.M > 8) return false;
    return q.M <= 4 ? W <= 16 * 4 * kGemv4MaxSeg : W <= 16 * kGemv4MaxSegTwo;
}

// Knobs at 2 force their kernel wherever it fits.  Returns a route or -1.
int forced_route(const RouteQuery &q) {
    if (knob(kGemvFine) >= 2 && q.fits_fine) return AP_ROUTE_FINE;
    if (knob(kGemvStream) >= 2 && q.fits_stream) return AP_ROUTE_STREAM;
    return -1;
}

// M = 1..4.  One route for the whole set.
int few_rows_route(const RouteQuery &q) {
    const int M = q.M, K = q.K, b = q.w_bits;
    const bool fine_ok = knob(kGemvFine) == 1 && q.fits_fine, stream_ok = knob(kGemvStream) == 1 && q.fits_stream;
    const int m4 = knob(kMatmulMfma4);
    // narrow linears (k/v projections with grouped heads) at 2..4 rows: the fine-grained kernel, 5-15 % on 1024 x 8192,
    // 5-9 % on 1024 x 4096 at 3-4 rows and up to 4 bits
    if (single(q) && fine_ok && q.lo <= 2048 && ((K >= 8192 && M >= 2) || (M >= 3 && b <= 4))) return AP_ROUTE_FINE;
    // long rows at 2..4 rows: gemv_kbit_kernel with four rows per workgroup (gemv_geometry shapes it so) wherever
    // long_rows_want_four says -- except M = 3 on rows of 8 waves or more at up to 4 bits (row-streaming kernel,
    // another 3-15 %; rows of 7 waves are 0-7 % faster with four rows) and M = 4 at 3 bits (4x4x4 kernel, 9 % on
    // 4096 x 14336 and 8192 x 28672)
    if (knob(kGemvRows) <= 0 && m4 <= 1 && q.geo->wpl == 1 && long_rows_want_four(M, K, b)) {
        if (single(q) && M == 3 && b <= 4 && q.geo->S >= 8 && stream_ok) return AP_ROUTE_STREAM;
        if (!(M == 4 && b == 3 && m4 == 1)) return AP_ROUTE_DOT;
    }
    if (single(q)) {
        // row-streaming kernel (fewest waves and instructions): 3-4 bits at two rows on rows of >= 8192 elements that
        // long_rows_want_four left alone (10-14 %).  It also served 3 bits at one row on wide linears (3-5 % then); since
        // the dot-product kernel's prologue was trimmed that kernel is 5-6 % faster there (11008 x 4096: 7.2 -> 6.8 us,
        // 14336 x 4096: 8.3 -> 7.8).
        if (stream_ok && M == 2 && K >= 8192 && b <= 4) return AP_ROUTE_STREAM;
        // fine-grained row-pair kernel (half the waves): 6-8 bits at four rows on rows of >= 8192 elements (6-15 %; at
        // 6 bits on rows of up to 12288 elements the 4x4x4 kernel is 13 % faster and takes over).  At one row it served
        // 6-7 bits on wide linears (11008 / 14336 x 4096; 3-6 % then): the dot-product kernel with two rows per workgroup is
        // now 3-6 % faster there (11008 x 4096 at 6 bits: 10.3 -> 9.7 us).
        if (fine_ok && M == 4 && K >= 8192 && b >= (K <= 12288 ? 7 : 6)) return AP_ROUTE_FINE;
    }
    // The 4x4x4 matrix-core kernel (cost per weight flat in M, one linear per launch): 3 and 4 rows on single linears with
    // enough rows to fill the chip, at up to 5 bits, and for 4 rows at every bit-width while a row fits one word
    // group per lane (K <= 8192; 6 bits up to 12288): 10-40 % faster than the dot-product kernel.  Not for sets (one
    // dot-product launch with four rows per workgroup beats a launch per member by 15-45 %) and not where
    // mid_rows_want_four says.
    if (m4 >= 1 && M >= 2 && mfma4_fits(q)) {
        if (m4 >= 2) return AP_ROUTE_MFMA4;
        const bool bits_ok = (M == 3 && b <= 5) || (M == 4 && (b <= 5 || K <= 8192 || (b == 6 && K <= 12288)));
        if (single(q) && !mid_rows_want_four(M, K, b) && bits_ok && q.rows >= 2048) return AP_ROUTE_MFMA4;
    }
    return AP_ROUTE_DOT;
}

// M = 5..8 under default knobs: where the dot-product kernel (cost linear in M, one launch for all members) still
// beats the matrix-core kernels (cost flat in M, one launch per member, 16 rows per workgroup):
//  - a linear of at most 2048 rows (k/v projections with grouped heads: 64-128 workgroups of the MFMA kernel): 10-54 %
//    faster at every M and bit-width; a set with such a member 6-50 % (at M >= 7 on rows of more than 4096 elements
//    only from 5 bits on);
//  - 7-8 bits on linears of >= 5120 rows of more than 4096 elements, where the MFMA kernel is at its worst (5120 x
//    5120, 13824 x 5120, 8192 x 8192, 28672 x 8192): 7-41 % at M = 5..7 at 8 bits (M = 8 too on rows of 5120
//    elements; M = 5 only on rows of 8193..16384: 5120 x 13824, 22 %; never beyond) and 9-20 % at M = 5 at 7 bits;
//    5120 x 5120 at M = 5 from 5 bits on (14-16 %);
//  - sets: at 8 bits on rows of 4097..8192 elements at every M (3-32 %); at M = 5 at 8 bits (8-46 %) and from 5 bits
//    on when no member has more than 8192 rows (15-37 %).
bool dot_beats_mfma(const RouteQuery &q) {
    const int M = q.M, K = q.K, b = q.w_bits;
    if (q.geo->wpl != 1) return false;
    if (single(q)) {
        if (q.lo <= 2048) return true;
        if (K <= 4096 || q.lo < 5120) return false;
        if (b == 8) return K <= 8192 ? (M <= 7 || K <= 5120) : (M == 5 && K <= 16384);
        if (b == 7) return M == 5 && K <= 8192;
        return M == 5 && b >= 5 && (long long)q.lo * K <= 32LL << 20;
    }
    if (q.lo <= 2048 && (M <= 6 || K <= 4096 || b >= 5)) return true;
    if (b == 8 && K > 4096 && K <= 8192) return true;
    if (M == 5 && K > 4096 && K <= 8192 && q.hi <= 8192) return true;  // q/k/v of the 13B model: 5-46 % at every bit-width
    return M == 5 && (b == 8 || (b >= 5 && q.hi <= 8192));
}

// M from the knob matmul_mfma_from on.  Routes per member (the matrix-core kernels serve one linear per launch).
void many_rows_route(const RouteQuery &q, int *route) {
    const int m4 = knob(kMatmulMfma4);
    const bool defaults = knob(kMatmulMfmaFrom) == 5 && m4 <= 1;
    if (defaults && q.M >= 5 && dot_beats_mfma(q)) {
        for (int g = 0; g < q.count; g++) route[g] = AP_ROUTE_DOT;
        return;
    }
    // 4x4x4 kernel with two groups of four activation rows (5..8 rows): on wide linears (16 rows per workgroup) with
    // rows of 3072..4096 elements (5..8 waves per workgroup) from 5 bits on it is 5-20 % faster than the 16x16x32
    // kernel; shorter and longer rows and narrower linears measured slower, and at 3 and 4 bits the 16x16x32 kernel
    // with its pair-table lookups is 4-18 % faster (11008 / 14336 x 4096; at 4 bits 6-12 % since its lookups run ahead
    // and its plane loads no longer wait).
    for (int g = 0; g < q.count; g++) {
        const bool pays = q.M >= 5 && q.K >= 3072 && q.N[g] >= 10240 && q.w_bits >= 5;
        route[g] = m4 >= 1 && mfma4_fits(q) && (m4 >= 2 || pays) ? AP_ROUTE_MFMA4 : AP_ROUTE_MFMA16;
    }
}

// route[g] = AP_ROUTE_* per member, and in *geo / *mem the geometry of the joint dot-product launch (used when every
// member has AP_ROUTE_DOT).  `out` may be null (route queries): the output pointers are then taken to be aligned.
int plan_matmul(int M, const int *N, int count, int K, int w_bits, uint16_t *const *out, GemvGeometry *geo,
                GemvMembers *mem, int *route) {
    const int rc = gemv_geometry(M, N, count, K, w_bits, geo, mem);
    if (rc != AP_OK && rc != AP_ELIMIT) return rc;
    auto all = [&](int r) {
        for (int g = 0; g < count; g++) route[g] = r;
        return AP_OK;
    };
    // a row longer than one workgroup of the dot-product kernel covers (65536 elements at M <= 2, 32768
    // beyond): the MFMA kernel walks rows of any length
    if (rc == AP_ELIMIT) return all(AP_ROUTE_MFMA16);
    RouteQuery q = {M, count, K, w_bits, N, N[0], N[0], 0, true, true, geo};
    for (int g = 0; g < count; g++) {
        const uint16_t *o = out ? out[g] : nullptr;
        q.lo = N[g] < q.lo ? N[g] : q.lo;
        q.hi = N[g] > q.hi ? N[g] : q.hi;
        q.rows += N[g];
        q.fits_fine = q.fits_fine && gemvf_fits(o, M, N[g], K);
        q.fits_stream = q.fits_stream && gemvp_fits(o, M, N[g], K);
    }
    const int forced = forced_route(q);
    if (forced >= 0)
        all(forced);
    else if (M < knob(kMatmulMfmaFrom))
        all(few_rows_route(q));
    else
        many_rows_route(q, route);
    // A set is either ONE dot-product launch or, member by member, exactly what each linear would get on its own
    // (a narrow k/v projection beside a wide q projection then still goes to the kernel that suits it).
    bool one_launch = true;
    for (int g = 0; g < count; g++) one_launch = one_launch && route[g] == AP_ROUTE_DOT;
    if (count > 1 && !one_launch) {
        for (int g = 0; g < count; g++) {
            GemvGeometry own;
            uint16_t *const *o = out ? out + g : nullptr;
            const int r = plan_matmul(M, N + g, 1, K, w_bits, o, &own, nullptr, route + g);
            if (r != AP_OK) return r;
        }
    }
    return AP_OK;
}

// Whether the fused GEMM (ap_gemm_kbit) beats dequant_kbit + a library GEMM for `M` activation rows.  Measured on the
// linear shapes of the Llama-2-7B / Llama-3-8B / 13B / 70B layers at 96..512 activation rows, every bit-width
// (fused / pair, us):
//  - always up to 32 activation rows (1.3-4x at 16);
//  - rows of a multiple of 128 elements (the tiled kernel), linears of at least 4096 rows: up to 128 activation rows at
//    every bit-width (11008 x 4096, 8 bits: 50 / 58; 28672 x 8192: 189 / 234; 5120 x 13824: 93 / 113); up to 256 at up to
//    5 bits (11008 x 4096, 4 bits: 58 / 73; 13824 x 5120, 5 bits: 79 / 97), at 6 bits except on linears of more than
//    16384 rows (28672 x 8192: 263 / 250), at 7 and 8 bits on linears of at most 8192 rows (8192 x 8192, 8 bits:
//    87 / 116; 5120 x 5120: 56 / 69; 4096 x 11008: 82 / 82; 11008 x 4096: 96 / 66); up to 512 at 3 bits on linears of
//    at most 8192 rows (4096 x 11008: 87 / 99; 8192 x 8192: 101 / 114; 14336 x 4096: 99 / 90);
//  - the same rows on linears of 1024..4095 rows: up to 512 activation rows at 3 and 4 bits (1024 x 4096: 11-15 /
//    18-23; at 6 bits and more the pair wins);
//  - other row lengths (the K-split kernel only): up to 64 on linears of fewer than 8192 rows, and on larger ones at up
//    to 5 bits -- except, on rows of more than 4096 elements, from 6 bits on linears of 5120 rows or more and from 5
//    bits on linears of at most 2048 rows; up to 128 on linears of 4096..8191 rows of at most 4096 elements.
// Beyond, one table lookup per weight and tile of activation rows costs more than materialising the weight once.
bool fused_gemm_pays(int M, int N, int K, int b) {
    if (M <= 32) return true;
    if ((K & 127) == 0 && M <= 512) {
        if (N >= 4096) {
            if (M <= 128) return true;
            if (M <= 256) return b <= 6 ? (b <= 5 || N <= 16384) : N <= 8192;
            return b == 3 && N <= 8192;
        }
        if (N >= 1024 && b <= 4) return true;
    }
    if (M <= 64) {
        if (K > 4096 && ((b >= 6 && N >= 5120) || (b >= 5 && N <= 2048))) return false;
        return N < 8192 || b <= 5;
    }
    return M <= kGemmMaxM && N >= 4096 && N < 8192 && K <= 4096;
}

// Whether ONE launch of the tiled GEMM over linears that share their input (ap_gemm_kbit_group) beats calling them one
// by one, each through whatever fused_gemm_pays picks (q/k/v and gate/up sets of the 7B / 8B / 13B layers at 16..256
// rows): from 33 rows on -- from 9 where every member has at most 8192 rows (q/k/v of the 7B layer at 16 rows, 3 bits:
// 16 us against 23; of the 13B layer: 20 against 36); wide members (gate/up) at 9..32 rows are as fast one by one -- up to
// 128 rows at every bit-width (q/k/v of the 7B layer at 128 rows, 3 bits: 33 us against 44 one by one and 128 for three
// dequant + GEMM pairs; gate/up at 8 bits: 96 against 115 for the pairs), up to 256 at up to 6 bits (gate/up at 5 bits:
// 105 against 145) and, at 7 and 8 bits, where every member has fewer than 8192 rows (q/k/v at 8 bits: 94 against 114;
// gate/up: 145 against 149); up to 512 at 3 bits where no member has more than 8192 rows, as each member alone would.
bool fused_set_pays(int M, const int *N, int count, int K, int b) {
    long long sum = 0;
    int hi = 0;
    for (int g = 0; g < count; g++) {
        sum += N[g];
        hi = N[g] > hi ? N[g] : hi;
    }
    if ((K & 127) != 0 || M <= 8 || M > 512 || sum < 4096) return false;
    if (M > 256) return b == 3 && hi <= 8192;
    if (M <= 32) return hi <= 8192 && K >= 1024;
    return M <= 128 || b <= 6 || hi < 8192;
}

}  // namespace

extern "C" {

int ap_matmul_kbit_swiglu(const uint16_t *x, const uint32_t *qweight_gate, const uint16_t *lut_gate,
                          const uint32_t *qweight_up, const uint16_t *lut_up, uint16_t *out, int M, int N, int K, int w_bits,
                          void *stream) {
    if (!x || !qweight_gate || !lut_gate || !qweight_up || !lut_up || !out) return AP_ENULL;
    const int rc = check_common(N, K, w_bits);
    if (rc != AP_OK) return rc;
    if (M < 1 || M > 4) return AP_EBATCH;
    if (!aligned16(x) || !aligned16(qweight_gate) || !aligned16(lut_gate) || !aligned16(qweight_up) || !aligned16(lut_up))
        return AP_EALIGN;
    GemvGeometry geo;
    geo.wpl = 1;
    geo.S = ((K >> 5) + kWave - 1) / kWave;
    geo.R = 2;
    geo.grid = N;  // one workgroup per (gate row, up row) pair
    if (geo.S > kGemvMaxSeg) return AP_ELIMIT;
    GemvMembers mem;
    memset(&mem, 0, sizeof mem);
    mem.qweight[0] = qweight_gate;
    mem.qweight[1] = qweight_up;
    mem.lut[0] = lut_gate;
    mem.lut[1] = lut_up;
    mem.out[0] = mem.out[1] = out;
    mem.n[0] = mem.n[1] = N;
    mem.wg_end[0] = mem.wg_end[1] = N;
    mem.count = 2;
    hipStream_t st = static_cast<hipStream_t>(stream);
    drain_stale_error();
    switch (w_bits) {
        case 3: launch_gemv_pair<3>(M, geo, x, mem, K, st); break;
        case 4: launch_gemv_pair<4>(M, geo, x, mem, K, st); break;
        case 5: launch_gemv_pair<5>(M, geo, x, mem, K, st); break;
        case 6: launch_gemv_pair<6>(M, geo, x, mem, K, st); break;
        case 7: launch_gemv_pair<7>(M, geo, x, mem, K, st); break;
        default: launch_gemv_pair<8>(M, geo, x, mem, K, st); break;
    }
    return launch_status();
}

// One launch of the tiled kernel over `count` linears (arguments already checked; geo from gemmt_geometry over all tiles).
int run_gemmt(const GemmtGeometry &geo, const uint16_t *x, int count, const uint32_t *const *qweight, const uint16_t *const *lut,
              uint16_t *const *out, const int *N, const long long *ldo, int M, int K, int w_bits, hipStream_t st) {
    GemmtMembers mem = {};
    mem.count = count;
    for (int g = 0; g < count; g++) {
        mem.qweight[g] = qweight[g];
        mem.lut[g] = lut[g];
        mem.out[g] = out[g];
        mem.N[g] = N[g];
        mem.ldo[g] = ldo ? ldo[g] : N[g];
        mem.tile0[g + 1] = mem.tile0[g] + (N[g] + 63) / 64;
    }
    switch (w_bits) {
        case 3: launch_gemmt<3>(geo, x, mem, M, K, st); break;
        case 4: launch_gemmt<4>(geo, x, mem, M, K, st); break;
        case 5: launch_gemmt<5>(geo, x, mem, M, K, st); break;
        case 6: launch_gemmt<6>(geo, x, mem, M, K, st); break;
        case 7: launch_gemmt<7>(geo, x, mem, M, K, st); break;
        default: launch_gemmt<8>(geo, x, mem, M, K, st); break;
    }
    return launch_status();
}

int ap_gemm_kbit(const uint16_t *x, const uint32_t *qweight, const uint16_t *lut, uint16_t *out, int M, int N, int K,
                 int w_bits, void *stream) {
    if (!x || !qweight || !lut || !out) return AP_ENULL;
    const int rc = check_common(N, K, w_bits);
    if (rc != AP_OK) return rc;
    if (M < 1) return AP_EBATCH;
    if (!aligned16(x) || !aligned16(qweight) || !aligned16(lut)) return AP_EALIGN;
    drain_stale_error();
    {
        GemmtGeometry tgeo;
        const int mode = knob(kGemmTiled);
        if (mode > 0 && gemmt_geometry(M, (N + 63) / 64, K, w_bits, &tgeo) && (mode >= 2 || gemmt_pays(M, N, K, w_bits)))
            return run_gemmt(tgeo, x, 1, &qweight, &lut, &out, &N, nullptr, M, K, w_bits, static_cast<hipStream_t>(stream));
    }
    // one launch serves up to kGemmMaxM activation rows; more go in chunks of that many, in order (the planes
    // are re-read per chunk; row offsets of 128 rows keep x and out 16-byte aligned for every K and N that passed)
    for (int m0 = 0; m0 < M; m0 += kGemmMaxM) {
        const int rows = M - m0 < kGemmMaxM ? M - m0 : kGemmMaxM;
        const int r = run_gemm(x + (size_t)m0 * K, qweight, lut, out + (size_t)m0 * N, rows, N, K, w_bits,
                               static_cast<hipStream_t>(stream));
        if (r != AP_OK) return r;
    }
    return AP_OK;
}

int ap_gemm_kbit_group(const uint16_t *x, int count, const uint32_t *const *qweight, const uint16_t *const *lut,
                       uint16_t *const *out, const int *N, const long long *ldo, int M, int K, int w_bits, void *stream) {
    if (!x || !qweight || !lut || !out || !N) return AP_ENULL;
    if (count < 1 || count > kGemmtMaxGroup) return AP_ELIMIT;
    if (M < 1) return AP_EBATCH;
    long long tiles = 0, rows = 0;  // tiles of all members; rows of the largest
    bool strided = false;
    for (int g = 0; g < count; g++) {
        if (!qweight[g] || !lut[g] || !out[g]) return AP_ENULL;
        const int rc = check_common(N[g], K, w_bits);
        if (rc != AP_OK) return rc;
        if (!aligned16(qweight[g]) || !aligned16(lut[g])) return AP_EALIGN;
        if (ldo && ldo[g] < N[g]) return AP_ESHAPE;
        strided = strided || (ldo && ldo[g] != N[g]);
        tiles += (N[g] + 63) / 64;
        rows = N[g] > rows ? N[g] : rows;
    }
    if (!aligned16(x)) return AP_EALIGN;
    drain_stale_error();
    GemmtGeometry tgeo;
    const int mode = knob(kGemmTiled);
    const bool fits = gemmt_geometry(M, tiles, K, w_bits, &tgeo);
    // Tiles of different members run side by side, and the launch costs about what its largest member alone would,
    // while the K-split kernel's launches add up: measured on the q/k/v and gate/up sets of the 7B / 8B / 13B layers at
    // 48..256 rows the one launch is 1.1-3x faster than the members one by one (q/k/v of the 7B layer at 128 rows,
    // 3 bits: 39 us against 69; of the 13B layer at 64 rows: 31 against 94) wherever there are more than 32 rows.  Sets
    // whose members all have fewer than 8192 rows (q/k/v) take it from 9 rows on, in tiles of 16 or 32 activation
    // At 9..32 rows, sets whose members have at most 8192 rows (q/k/v) take it too, in tiles of 16 or 32 activation rows
    // (7B q/k/v at 16 rows: 16-24 us against 23-26 at 3-5 bits; 13B: 20-40 against 36-68; 70B: 21-48 against 39-64); wide
    // members (gate/up) are within 10 % either way one by one.
    const bool pays = M > 32 || (M > 8 && rows <= 8192 && K >= 1024);
    if (fits && (strided || (count > 1 && mode > 0 && (mode >= 2 || pays))))
        return run_gemmt(tgeo, x, count, qweight, lut, out, N, ldo, M, K, w_bits, static_cast<hipStream_t>(stream));
    // only the tiled kernel writes rows that are not dense: rows it cannot walk at all are a shape error, a size or a
    // forced tile beyond its geometry a limit (the caller may still ask for dense results)
    if (strided) return (K & 127) != 0 ? AP_ESHAPE : AP_ELIMIT;
    for (int g = 0; g < count; g++) {
        const int r = ap_gemm_kbit(x, qweight[g], lut[g], out[g], M, N[g], K, w_bits, stream);
        if (r != AP_OK) return r;
    }
    return AP_OK;
}

int ap_matmul_kbit(const uint16_t *x, const uint32_t *qweight, const uint16_t *lut, uint16_t *out, int M, int N,
                   int K, int w_bits, void *stream) {
    return ap_matmul_kbit_group(x, 1, &qweight, &lut, &out, &N, M, K, w_bits, stream);
}

int ap_matmul_kbit_group(const uint16_t *x, int count, const uint32_t *const *qweight, const uint16_t *const *lut,
                         uint16_t *const *out, const int *N, int M, int K, int w_bits, void *stream) {
    if (!x || !qweight || !lut || !out || !N) return AP_ENULL;
    if (count < 1 || count > kGemvMaxGroup) return AP_ELIMIT;
    for (int g = 0; g < count; g++)
        if (!qweight[g] || !lut[g] || !out[g]) return AP_ENULL;
    GemvGeometry geo;
    GemvMembers mem = {};
    int route[kGemvMaxGroup];
    const int rc = plan_matmul(M, N, count, K, w_bits, out, &geo, &mem, route);
    if (rc != AP_OK) return rc;
    if (!aligned16(x)) return AP_EALIGN;
    for (int g = 0; g < count; g++) {
        if (!aligned16(qweight[g]) || !aligned16(lut[g])) return AP_EALIGN;
        mem.qweight[g] = qweight[g];
        mem.lut[g] = lut[g];
        mem.out[g] = out[g];
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    drain_stale_error();
    bool one_launch = true;
    for (int g = 0; g < count; g++) one_launch = one_launch && route[g] == AP_ROUTE_DOT;
    if (count > 1 && !one_launch) {  // member by member, each as a linear of its own
        for (int g = 0; g < count; g++) {
            const int r = ap_matmul_kbit_group(x, 1, qweight + g, lut + g, out + g, N + g, M, K, w_bits, stream);
            if (r != AP_OK) return r;
        }
        return AP_OK;
    }
    if (one_launch) {  // the whole set in one launch
        switch (w_bits) {
            case 3: launch_gemv<3>(M, geo, x, mem, K, st); break;
            case 4: launch_gemv<4>(M, geo, x, mem, K, st); break;
            case 5: launch_gemv<5>(M, geo, x, mem, K, st); break;
            case 6: launch_gemv<6>(M, geo, x, mem, K, st); break;
            case 7: launch_gemv<7>(M, geo, x, mem, K, st); break;
            default: launch_gemv<8>(M, geo, x, mem, K, st); break;
        }
        return launch_status();
    }
    for (int g = 0; g < count; g++) {
        int r;
        switch (route[g]) {
            case AP_ROUTE_STREAM: r = run_gemvp(x, qweight[g], lut[g], out[g], M, N[g], K, w_bits, st); break;
            case AP_ROUTE_FINE: r = run_gemvf(x, qweight[g], lut[g], out[g], M, N[g], K, w_bits, st); break;
            case AP_ROUTE_MFMA4: r = run_gemv4(x, qweight[g], lut[g], out[g], M, N[g], K, w_bits, st); break;
            default: r = run_gemm(x, qweight[g], lut[g], out[g], M, N[g], K, w_bits, st); break;
        }
        if (r != AP_OK) return r;
    }
    return AP_OK;
}

int ap_gemm_kbit_pays(int M, int N, int K, int w_bits) {
    const int rc = check_common(N, K, w_bits);
    if (rc != AP_OK) return rc;
    if (M < 1) return AP_EBATCH;
    return fused_gemm_pays(M, N, K, w_bits) ? 1 : 0;
}

int ap_gemm_kbit_group_pays(int count, const int *N, int M, int K, int w_bits) {
    if (!N) return AP_ENULL;
    if (count < 1 || count > kGemmtMaxGroup) return AP_ELIMIT;
    for (int g = 0; g < count; g++) {
        const int rc = check_common(N[g], K, w_bits);
        if (rc != AP_OK) return rc;
    }
    if (M < 1) return AP_EBATCH;
    return fused_set_pays(M, N, count, K, w_bits) ? 1 : 0;
}

int ap_matmul_kbit_route(int M, int N, int K, int w_bits, int *route) {
    if (!route) return AP_ENULL;
    GemvGeometry geo;
    return plan_matmul(M, &N, 1, K, w_bits, nullptr, &geo, nullptr, route);
}

int ap_matmul_kbit_group_route(int count, const int *N, int M, int K, int w_bits, int *route, int *rows) {
    if (!N || !route) return AP_ENULL;
    if (count < 1 || count > kGemvMaxGroup) return AP_ELIMIT;
    GemvGeometry geo = {};  // rows stays 0 when no dot-product launch can serve the set
    const int rc = plan_matmul(M, N, count, K, w_bits, nullptr, &geo, nullptr, route);
    if (rc == AP_OK && rows) *rows = geo.R;
    return rc;
}

}  // extern "C"

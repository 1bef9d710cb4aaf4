// C ABI of libanyprec_hip: argument checks, launch geometry, dispatch.
// The declarations and their reference counterparts are in include/anyprec_hip.h.
#include <hip/hip_runtime.h>
#include <stdlib.h>

#include "anyprec_hip.h"
#include "ap_dequant.hpp"
#include "ap_gemm_launch.hpp"
#include "ap_gemv4_launch.hpp"
#include "ap_gemv_launch.hpp"

namespace {

using namespace ap;

constexpr int kNumCUs = 256;  // MI355X: 8 XCDs x 32 CUs

struct Tuning {
    int target_waves;  // waves the GEMV grid aims for (rows per wave follows)
    int force_rows;    // > 0: rows per wave, overrides target_waves
    int force_wpl;     // > 0: words per lane
    int dequant_blocks_per_cu;
    int mfma_from_rows;     // ap_matmul_kbit uses the MFMA kernel from this many activation rows on
    int force_gemm_split;   // > 0: K-split waves per workgroup of the fused GEMM
    int mfma4_mode;         // 4x4x4 matrix-core kernel: 0 never, 1 where it pays, 2 for 2..8 rows wherever it fits
    int force_gemv4_groups; // > 0: word groups per wave of that kernel
    int gemm_rb2_mode;      // fused GEMM, two weight-row blocks per workgroup: 0 never, 1 where it pays, 2 always
};

int env_int(const char *name, int dflt) {
    const char *v = getenv(name);
    return (v && *v) ? atoi(v) : dflt;
}

const Tuning &tuning() {
    static const Tuning t = {
        env_int("AP_GEMV_TARGET_WAVES", 16384),
        env_int("AP_GEMV_ROWS", 0),
        env_int("AP_GEMV_WPL", 0),
        env_int("AP_DEQUANT_BLOCKS_PER_CU", 32),
        env_int("AP_MATMUL_MFMA_FROM", 5),
        env_int("AP_GEMM_SPLIT", 0),
        env_int("AP_MATMUL_MFMA4", 1),
        env_int("AP_GEMV4_GROUPS", 0),
        env_int("AP_GEMM_RB2", 1),
    };
    return t;
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

int check_common(int N, int K, int w_bits) {
    if (w_bits < 3 || w_bits > 8) return AP_EBITS;
    if (N < 1 || K < 32 || (K & 31) != 0) return AP_ESHAPE;
    return AP_OK;
}

// Launch geometry for `count` linears of n[0..count) rows that share K, M and w_bits.
int gemv_geometry(int M, const int *n, int count, int K, int w_bits, GemvGeometry *geo, GemvMembers *mem) {
    long long rows = 0;
    for (int g = 0; g < count; g++) {
        const int rc = check_common(n[g], K, w_bits);
        if (rc != AP_OK) return rc;
        rows += n[g];
    }
    if (M < 1 || M > 8) return AP_EBATCH;
    const Tuning &t = tuning();
    const int W = K >> 5;
    // One word per lane (two waves per 4096 elements of a row) measured 5-15 % faster than
    // two on planes that come from HBM, up to rows of 16384 elements; beyond (more than 8 waves
    // per row) two words per lane are 7-10 % faster (8192 x 28672), and they are needed when
    // one word per lane would take more waves than a workgroup holds.
    int wpl = 1;
    if (M <= 2 && (W & 1) == 0 && (W + kWave - 1) / kWave > 8) wpl = 2;
    if (t.force_wpl == 1 || (t.force_wpl == 2 && (W & 1) == 0 && M <= 2)) wpl = t.force_wpl;
    const int seg = kWave * wpl;
    const int S = (W + seg - 1) / seg;
    if (S > kGemvMaxSeg) return AP_ELIMIT;
    // One row per workgroup until that would launch more than target_waves waves, then two
    // (the second row reuses the activation registers; more rows lengthen the compute
    // tail).  From M = 3 on the activations are the larger load: always two rows.
    int R = t.force_rows > 0 ? t.force_rows : (int)((rows * S + t.target_waves - 1) / t.target_waves);
    R = (R >= 2 || M > 2) ? 2 : 1;
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

template <int BITS>
void launch_dequant(const uint32_t *qweight, const uint16_t *lut, uint16_t *out, int N, int K, hipStream_t stream) {
    const int S = ((K >> 5) + kWave - 1) / kWave;  // 64-word segments per row
    long long blocks = ((long long)N * S + kDequantWaves - 1) / kDequantWaves;
    const long long cap = (long long)kNumCUs * tuning().dequant_blocks_per_cu;
    if (blocks > cap) blocks = cap;
    dequant_kbit_kernel<BITS><<<dim3((unsigned)blocks), dim3(kDequantWaves * kWave), 0, stream>>>(
        qweight, reinterpret_cast<const half_t *>(lut), reinterpret_cast<half_t *>(out), N, K);
}

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
        default: break;
    }
    if (code > 0) return hipGetErrorString((hipError_t)code);
    return "unknown error code";
}

int ap_dequant_kbit(const uint32_t *qweight, const uint16_t *lut, uint16_t *out, int N, int K, int w_bits,
                    void *stream) {
    if (!qweight || !lut || !out) return AP_ENULL;
    const int rc = check_common(N, K, w_bits);
    if (rc != AP_OK) return rc;
    if (!aligned16(qweight) || !aligned16(lut) || !aligned16(out)) return AP_EALIGN;
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (w_bits) {
        case 3: launch_dequant<3>(qweight, lut, out, N, K, st); break;
        case 4: launch_dequant<4>(qweight, lut, out, N, K, st); break;
        case 5: launch_dequant<5>(qweight, lut, out, N, K, st); break;
        case 6: launch_dequant<6>(qweight, lut, out, N, K, st); break;
        case 7: launch_dequant<7>(qweight, lut, out, N, K, st); break;
        default: launch_dequant<8>(qweight, lut, out, N, K, st); break;
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

// Launch of the fused dequant -> MFMA kernel (arguments already checked).
int run_gemm(const uint16_t *x, const uint32_t *qweight, const uint16_t *lut, uint16_t *out, int M, int N, int K,
             int w_bits, hipStream_t st) {
    // the kernel addresses the activations with 32-bit byte offsets
    if ((long long)M * K * 2 > 0xffffffffLL) return AP_ELIMIT;
    GemmGeometry geo;
    geo.mb = (M + 15) / 16;
    const int W = K >> 5;
    // Two blocks of 16 weight rows per workgroup halve the L2 traffic of the activations, which
    // bounds this kernel, but also the number of workgroups, and they need twice the plane
    // registers: measured faster from 9 activation rows on, on linears of at least 8192 rows -- at
    // 3 bits, and at up to 5 bits (6 with two activation row blocks) when the linear has at least
    // 56 M weights (14336 x 4096, 8192 x 8192, 28672 x 8192: 5-25 %).
    const int rb_mode = tuning().gemm_rb2_mode;  // 0 never, 1 where it pays, 2 wherever the kernel allows
    const bool rb_fits = (W & 3) == 0 && N >= 32;
    const bool rb_pays = M > 8 && N >= 8192 &&
                         (w_bits == 3 || (w_bits <= (geo.mb >= 2 ? 6 : 5) && (long long)N * K >= 56LL << 20));
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
    int ks = tuning().force_gemm_split > 0 ? tuning().force_gemm_split : kGemmMaxSplit;
    if (ks > kGemmMaxSplit) ks = kGemmMaxSplit;
    if (ks > steps) ks = steps;
    if (ks < 1) ks = 1;
    geo.ks = ks;
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

int run_gemv4(const uint16_t *x, const uint32_t *qweight, const uint16_t *lut, uint16_t *out, int M, int N, int K,
              int w_bits, hipStream_t st) {
    Gemv4Geometry geo;
    if (M > 8) return AP_EBATCH;
    const int W = K >> 5;
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
        int G = tuning().force_gemv4_groups > 0 ? tuning().force_gemv4_groups : 1;
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

}  // namespace

extern "C" {

int ap_gemm_kbit(const uint16_t *x, const uint32_t *qweight, const uint16_t *lut, uint16_t *out, int M, int N, int K,
                 int w_bits, void *stream) {
    if (!x || !qweight || !lut || !out) return AP_ENULL;
    const int rc = check_common(N, K, w_bits);
    if (rc != AP_OK) return rc;
    if (M < 1 || M > kGemmMaxM) return AP_EBATCH;
    if (!aligned16(x) || !aligned16(qweight) || !aligned16(lut)) return AP_EALIGN;
    return run_gemm(x, qweight, lut, out, M, N, K, w_bits, static_cast<hipStream_t>(stream));
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
    const int rc = gemv_geometry(M, N, count, K, w_bits, &geo, &mem);
    if (rc != AP_OK && rc != AP_ELIMIT) return rc;
    if (!aligned16(x)) return AP_EALIGN;
    for (int g = 0; g < count; g++) {
        if (!aligned16(qweight[g]) || !aligned16(lut[g])) return AP_EALIGN;
        mem.qweight[g] = qweight[g];
        mem.lut[g] = lut[g];
        mem.out[g] = out[g];
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (rc == AP_ELIMIT) {
        // a row longer than one workgroup of the dot-product kernel covers (65536 elements at M <= 2,
        // 32768 beyond): the MFMA kernel walks rows of any length
        for (int g = 0; g < count; g++) {
            const int r = run_gemm(x, qweight[g], lut[g], out[g], M, N[g], K, w_bits, st);
            if (r != AP_OK) return r;
        }
        return AP_OK;
    }
    // The 4x4x4 matrix-core kernel, whose cost per weight does not grow with M, where it measured
    // faster than both other kernels (it serves one linear per launch):
    //  - 3 and 4 activation rows on linears with enough rows to fill the chip (8 per workgroup), at up
    //    to 5 bits, and for 4 rows at every bit-width while a row fits one word group per lane
    //    (K <= 8192): 10-40 % faster than the dot-product kernel;
    //  - 5..8 activation rows on wide linears (16 rows per workgroup) with rows of 3072..4096 elements
    //    (5..8 waves per workgroup): 5-20 % faster than the 16x16x32 MFMA kernel.  Shorter and longer
    //    rows and narrower linears measured slower.
    const int m4 = tuning().mfma4_mode;
    long long rows = 0;
    for (int g = 0; g < count; g++) rows += N[g];
    auto use4 = [&](int n) {
        const int W = K >> 5;
        if (m4 == 0 || M < 2 || M > 8) return false;
        if (M <= 4) {  // decided for the group as a whole, by its mean row count
            if (W > 16 * 4 * kGemv4MaxSeg) return false;  // at most 4 word groups per wave, 16 waves
            if (m4 >= 2) return true;
            return ((M == 3 && w_bits <= 5) || (M == 4 && (w_bits <= 5 || K <= 8192))) && rows >= 2048LL * count;
        }
        if (W > 16 * kGemv4MaxSegTwo) return false;
        if (m4 >= 2) return true;
        return K >= 3072 && n >= 10240;  // per member; the others go to the MFMA kernel
    };
    bool any4 = false;
    for (int g = 0; g < count; g++) any4 |= use4(N[g]);
    if (any4) {
        for (int g = 0; g < count; g++) {
            const int r = use4(N[g]) ? run_gemv4(x, qweight[g], lut[g], out[g], M, N[g], K, w_bits, st)
                                     : run_gemm(x, qweight[g], lut[g], out[g], M, N[g], K, w_bits, st);
            if (r != AP_OK) return r;
        }
        return AP_OK;
    }
    // From 5 activation rows on, the 16x16x32 MFMA kernel (cost flat in M up to 16 rows) is faster than
    // the dot-product kernel (cost linear in M) on most shapes and bit-widths; one linear per launch.
    if (M >= tuning().mfma_from_rows) {
        for (int g = 0; g < count; g++) {
            const int r = run_gemm(x, qweight[g], lut[g], out[g], M, N[g], K, w_bits, st);
            if (r != AP_OK) return r;
        }
        return AP_OK;
    }
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

}  // extern "C"

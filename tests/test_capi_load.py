"""The C-ABI library loads and exports every function include/*.h declares
(CPU only: no compute entry point is launched here)."""
import ctypes
import glob
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "any-precision-llm_amd", "lib", "libanyprec_hip.so")


def _declared_functions():
    names = []
    for hdr in glob.glob(os.path.join(ROOT, "include", "*.h")):
        text = re.sub(r"/\*.*?\*/", "", open(hdr).read(), flags=re.S)
        names += re.findall(r"\b(ap_[a-z0-9_]+)\s*\(", text)
    return sorted(set(names))


def test_header_declares_the_boundary():
    names = _declared_functions()
    for must in ("ap_dequant_kbit", "ap_matmul_kbit", "ap_strerror", "ap_abi_version"):
        assert must in names


def test_library_exports_every_declared_symbol():
    assert os.path.exists(LIB), "build libanyprec_hip.so first (python any-precision-llm_amd/build.py)"
    lib = ctypes.CDLL(LIB)
    for name in _declared_functions():
        assert hasattr(lib, name), name


def test_binding_lists_every_declared_symbol():
    from any_precision_amd import _capi
    assert sorted(_capi.EXPORTS) == _declared_functions()
    assert _capi.lib.ap_abi_version() == _capi.AP_ABI_VERSION


def test_strerror_and_argument_errors_need_no_gpu():
    from any_precision_amd import _capi
    L = _capi.lib
    assert _capi.strerror(0) == "ok"
    for code in (-1, -2, -3, -4, -5, -6, -7):
        assert _capi.strerror(code) not in ("ok", "unknown error code")
    fake = 4096  # non-null, 16-byte aligned; argument errors return before any launch
    assert L.ap_dequant_kbit(None, fake, fake, 4, 64, 3, None) == _capi.AP_ENULL
    assert L.ap_dequant_kbit(fake, fake, fake, 4, 64, 2, None) == _capi.AP_EBITS
    assert L.ap_dequant_kbit(fake, fake, fake, 4, 64, 9, None) == _capi.AP_EBITS
    assert L.ap_dequant_kbit(fake, fake, fake, 4, 48, 3, None) == _capi.AP_ESHAPE
    assert L.ap_dequant_kbit(fake, fake, fake, 0, 64, 3, None) == _capi.AP_ESHAPE
    assert L.ap_dequant_kbit(fake, fake, fake + 8, 4, 64, 3, None) == _capi.AP_EALIGN
    assert L.ap_matmul_kbit(fake, fake, fake, None, 1, 4, 64, 3, None) == _capi.AP_ENULL
    assert L.ap_matmul_kbit(fake, fake, fake, fake, 0, 4, 64, 3, None) == _capi.AP_EBATCH
    assert L.ap_matmul_kbit(fake, fake, fake, fake, 9, 4, 64, 3, None) == _capi.AP_EBATCH
    assert L.ap_matmul_kbit(fake + 2, fake, fake, fake, 1, 4, 64, 3, None) == _capi.AP_EALIGN
    assert L.ap_matmul_kbit(fake, fake, fake, fake, 1, 4, 64, 11, None) == _capi.AP_EBITS
    with pytest.raises(ValueError):
        _capi.check(_capi.AP_EBITS, "x")
    with pytest.raises(RuntimeError):
        _capi.check(98, "x")


def test_decode_step_argument_errors_need_no_gpu():
    from any_precision_amd import _capi
    L = _capi.lib
    fake = 4096
    assert L.ap_add_rmsnorm(None, None, fake, fake, fake, 1, 128, 1e-5, None) == _capi.AP_ENULL
    assert L.ap_add_rmsnorm(fake, None, fake, fake, fake, 0, 128, 1e-5, None) == _capi.AP_ESHAPE
    assert L.ap_add_rmsnorm(fake, None, fake, fake, fake, 1, 100, 1e-5, None) == _capi.AP_ESHAPE
    assert L.ap_add_rmsnorm(fake, fake + 2, fake, fake, fake, 1, 128, 1e-5, None) == _capi.AP_EALIGN
    sw = lambda **kw: L.ap_matmul_kbit_swiglu(*[kw.get(k, d) for k, d in (
        ("x", fake), ("qg", fake), ("lg", fake), ("qu", fake), ("lu", fake), ("out", fake), ("M", 1), ("N", 8), ("K", 64),
        ("b", 3), ("stream", None))])
    assert sw(qu=None) == _capi.AP_ENULL
    assert sw(M=5) == _capi.AP_EBATCH
    assert sw(b=9) == _capi.AP_EBITS
    assert sw(K=40) == _capi.AP_ESHAPE
    assert sw(K=32 * 64 * 17) == _capi.AP_ELIMIT          # more than 16 waves per row
    assert sw(lg=fake + 4) == _capi.AP_EALIGN
    assert L.ap_decode_advance(fake, 100, fake, None, fake, 64, None) == _capi.AP_ENULL
    assert L.ap_decode_advance(fake, 0, fake, fake, fake, 64, None) == _capi.AP_ESHAPE
    assert L.ap_decode_advance(fake + 2, 100, fake, fake, fake, 64, None) == _capi.AP_EALIGN
    assert L.ap_silu_mul(fake, None, fake, 64, None) == _capi.AP_ENULL
    assert L.ap_silu_mul(fake, fake, fake, 12, None) == _capi.AP_ESHAPE
    assert L.ap_silu_mul(fake, fake, fake + 4, 64, None) == _capi.AP_EALIGN
    att = lambda **kw: L.ap_decode_attention(*[kw.get(k, d) for k, d in (
        ("qkv", fake), ("cos", fake), ("sin", fake), ("kc", fake), ("vc", fake), ("pos", fake), ("out", fake),
        ("nh", 8), ("nkv", 2), ("hd", 128), ("max_len", 512), ("scale", 0.1), ("stream", None))])
    assert att(pos=None) == _capi.AP_ENULL
    assert att(nkv=3) == _capi.AP_ESHAPE          # query heads must be a multiple of the key/value heads
    assert att(hd=96) == _capi.AP_ESHAPE
    assert att(max_len=8193) == _capi.AP_ELIMIT
    assert att(kc=fake + 8) == _capi.AP_EALIGN


def test_gemm_group_argument_errors_need_no_gpu():
    from any_precision_amd import _capi
    fake = 4096
    call = lambda **kw: _capi.gemm_group(kw.get("x", fake), kw.get("q", [fake, fake]), kw.get("t", [fake, fake]),
                                         kw.get("o", [fake, fake]), kw.get("N", [64, 64]), kw.get("ldo"), kw.get("M", 40),
                                         kw.get("K", 128), kw.get("b", 3), 0)
    assert call(x=None) == _capi.AP_ENULL and call(q=[fake, None]) == _capi.AP_ENULL
    assert call(q=[fake] * 5, t=[fake] * 5, o=[fake] * 5, N=[64] * 5) == _capi.AP_ELIMIT
    assert call(M=0) == _capi.AP_EBATCH
    assert call(b=2) == _capi.AP_EBITS
    assert call(K=100) == _capi.AP_ESHAPE and call(N=[64, 0]) == _capi.AP_ESHAPE
    assert call(ldo=[128, 63]) == _capi.AP_ESHAPE          # rows of a result overlap
    assert call(t=[fake, fake + 2]) == _capi.AP_EALIGN and call(x=fake + 8) == _capi.AP_EALIGN


def test_dequant_group_and_pays_argument_errors_need_no_gpu():
    """ap_dequant_kbit_group, ap_gemm_kbit_pays and ap_gemm_kbit_group_pays check their arguments before any HIP call."""
    import ctypes
    from any_precision_amd import _capi
    fake = 4096
    call = lambda **kw: _capi.dequant_group(kw.get("q", [fake, fake]), kw.get("t", [fake, fake]), kw.get("o", [fake, fake]),
                                            kw.get("N", [64, 8]), kw.get("K", [128, 2080]), kw.get("b", 3), 0)
    assert call(q=[fake, None]) == _capi.AP_ENULL and call(o=[None, fake]) == _capi.AP_ENULL
    assert call(q=[fake] * 9, t=[fake] * 9, o=[fake] * 9, N=[64] * 9, K=[128] * 9) == _capi.AP_ELIMIT
    assert _capi.lib.ap_dequant_kbit_group(0, None, None, None, None, None, 3, None) == _capi.AP_ENULL
    assert call(b=9) == _capi.AP_EBITS
    assert call(K=[128, 100]) == _capi.AP_ESHAPE and call(N=[64, 0]) == _capi.AP_ESHAPE
    assert call(t=[fake, fake + 2]) == _capi.AP_EALIGN and call(o=[fake + 8, fake]) == _capi.AP_EALIGN
    assert _capi.lib.ap_dequant_kbit(None, fake, fake, 8, 64, 3, None) == _capi.AP_ENULL      # the single call is a set of one
    assert _capi.lib.ap_gemm_kbit_pays(16, 4096, 4096, 3) == 1 and _capi.lib.ap_gemm_kbit_pays(16384, 4096, 4096, 3) == 0
    assert _capi.lib.ap_gemm_kbit_pays(0, 4096, 4096, 3) == _capi.AP_EBATCH
    assert _capi.lib.ap_gemm_kbit_pays(16, 4096, 4100, 3) == _capi.AP_ESHAPE
    assert _capi.lib.ap_gemm_kbit_pays(16, 4096, 4096, 2) == _capi.AP_EBITS
    three = (ctypes.c_int * 3)(4096, 4096, 4096)
    assert _capi.lib.ap_gemm_kbit_group_pays(3, three, 128, 4096, 3) == 1
    assert _capi.lib.ap_gemm_kbit_group_pays(3, three, 8, 4096, 3) == 0
    assert _capi.lib.ap_gemm_kbit_group_pays(5, three, 128, 4096, 3) == _capi.AP_ELIMIT
    assert _capi.lib.ap_gemm_kbit_group_pays(3, None, 128, 4096, 3) == _capi.AP_ENULL
    with pytest.raises(ValueError):
        _capi.gemm_pays(16, 0, 4096, 3)


def test_geometry_covers_rows_and_words():
    from any_precision_amd import _capi
    for M in (1, 2, 4, 8):
        for N, K in ((4096, 4096), (11008, 4096), (4096, 11008), (1024, 4096), (4096, 14336), (7, 32), (5, 2080)):
            g = _capi.matmul_geometry(M, N, K, 4)
            W = K // 32
            assert g["segments"] * 64 * g["wpl"] >= W and W % g["wpl"] == 0
            assert g["segments"] <= 16 and 1 <= g["rows"] <= 16
            assert g["grid"] * g["rows"] >= N and (g["grid"] - 1) * g["rows"] < N
    with pytest.raises(ValueError):
        _capi.matmul_geometry(1, 4, 32 * 64 * 2 * 17, 4)     # more K-segments than a workgroup holds


def test_tuning_knobs_need_no_gpu():
    """ap_set_tuning / ap_get_tuning only touch the library's knob table."""
    from any_precision_amd import _capi
    assert _capi.lib.ap_set_tuning(None, 1) == _capi.AP_ENULL
    assert _capi.lib.ap_set_tuning(b"no_such_knob", 1) == _capi.AP_EKNOB
    with pytest.raises(ValueError):
        _capi.get_tuning("no_such_knob")
    for name in ("gemv_target_waves", "gemv_rows", "gemv_wpl", "dequant_blocks_per_cu", "matmul_mfma_from", "gemm_split",
                 "matmul_mfma4", "gemv4_groups", "gemm_rb2", "gemv_stream", "gemv_stream_waves", "gemv_fine",
                 "gemm_walk", "gemm_walk_wgs", "gemm_tiled", "gemm_tile", "gemm_tile_split", "gemm_lookahead"):
        before = _capi.get_tuning(name)
        with _capi.tuning(**{name: before + 3}):
            assert _capi.get_tuning(name) == before + 3
        assert _capi.get_tuning(name) == before
    # the geometry report follows the knobs at once: nothing is cached
    with _capi.tuning(gemv_rows=2):
        assert _capi.matmul_geometry(1, 4096, 4096, 4)["rows"] == 2
    assert _capi.matmul_geometry(1, 4096, 4096, 4)["rows"] == 1


def test_route_report_follows_the_rule_and_the_knobs():
    """ap_matmul_kbit_route names the kernel a single linear gets; forcing knobs change it at once."""
    from any_precision_amd import _capi
    assert _capi.matmul_route(1, 4096, 4096, 4) == "dot"
    assert _capi.matmul_route(1, 11008, 4096, 3) == "dot"
    assert _capi.matmul_route(1, 11008, 4096, 7) == "dot" and _capi.matmul_route(4, 4096, 11008, 7) == "fine"
    assert _capi.matmul_route(1, 11008, 4096, 8) == "dot"
    assert _capi.matmul_geometry(1, 11008, 4096, 8)["rows"] == 1        # one row per workgroup at 8 bits
    assert _capi.matmul_route(1, 4096, 11008, 3) == "dot"
    assert _capi.matmul_route(2, 4096, 14336, 4) == "dot" and _capi.matmul_geometry(2, 4096, 14336, 4)["rows"] == 4
    assert _capi.matmul_route(2, 8192, 28672, 4) == "stream"           # rows of 14 waves keep the streaming kernel
    assert _capi.matmul_geometry(2, 4096, 4096, 3)["rows"] == 2 and _capi.matmul_geometry(2, 4096, 4096, 5)["rows"] == 1
    assert _capi.matmul_route(8, 4096, 4096, 4) == "mfma16"
    assert _capi.matmul_route(8, 14336, 4096, 5) == "mfma4" and _capi.matmul_route(8, 14336, 4096, 4) == "mfma16"
    assert _capi.matmul_route(8, 14336, 4096, 3) == "mfma16"            # pair-table lookups: faster at 3 bits
    assert _capi.matmul_route(8, 1024, 4096, 3) == "dot"                # too few rows for 16 per workgroup
    assert _capi.matmul_route(5, 5120, 5120, 8) == "dot" and _capi.matmul_route(8, 8192, 8192, 8) == "mfma16"
    assert _capi.matmul_route(5, 8192, 28672, 8) == "mfma16" and _capi.matmul_route(3, 1024, 8192, 5) == "fine"
    # sets of linears (ap_matmul_kbit_group): one dot-product launch up to 4 rows, four weight rows per workgroup at 3-4
    assert _capi.matmul_group_route(1, [4096, 4096, 4096], 4096, 3) == (["dot"] * 3, 4)
    assert _capi.matmul_group_route(1, [4096, 4096, 4096], 4096, 8) == (["dot"] * 3, 1)
    assert _capi.matmul_group_route(3, [4096, 1024, 1024], 4096, 5) == (["dot"] * 3, 4)
    assert _capi.matmul_group_route(8, [4096, 1024, 1024], 4096, 3)[0] == ["dot"] * 3       # a narrow member
    assert _capi.matmul_group_route(8, [11008, 11008], 4096, 5)[0] == ["mfma4", "mfma4"]     # a launch per member
    assert _capi.matmul_group_route(8, [4096, 4096, 4096], 4096, 3)[0] == ["mfma16"] * 3
    assert _capi.matmul_group_route(8, [8192, 1024, 1024], 8192, 3)[0] == ["mfma16", "dot", "dot"]   # each as a linear of its own
    with pytest.raises(ValueError):
        _capi.matmul_group_route(1, [64] * 5, 4096, 3)
    with _capi.tuning(matmul_mfma_from=5, matmul_mfma4=2):
        assert _capi.matmul_route(8, 1024, 4096, 3) != "dot"            # a forced kernel overrides the rule
    assert _capi.matmul_route(1, 8, 32 * 64 * 2 * 17, 4) == "mfma16"      # longer than a workgroup covers
    with _capi.tuning(gemv_stream=0, gemv_fine=0):
        assert _capi.matmul_route(1, 11008, 4096, 3) == "dot"
    with _capi.tuning(gemv_stream=2):
        assert _capi.matmul_route(3, 64, 4096, 5) == "stream"
        assert _capi.matmul_route(3, 64, 4128, 5) != "stream"             # rows must be a multiple of 128 elements
    with _capi.tuning(gemv_fine=2):
        assert _capi.matmul_route(1, 63, 4096, 5) == "dot"                # odd row count: not served
    with pytest.raises(ValueError):
        _capi.matmul_route(9, 64, 4096, 5)

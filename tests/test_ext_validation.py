"""Argument validation of the drop-in ops (CPU only: every case raises before a launch)."""
import pytest
import torch

import any_precision_ext as ext


def _w(planes=8, N=4, W=2, b=3):
    return torch.zeros((planes, N, W), dtype=torch.int32), torch.zeros((N, 1 << b), dtype=torch.float16)


def test_op_names_and_signatures():
    import inspect
    assert list(inspect.signature(ext.matmul_kbit).parameters)[1:] == ["qweight", "lut", "w_bits"]
    assert list(inspect.signature(ext.dequant_kbit).parameters) == ["qweight", "lut", "w_bits"]


@pytest.mark.parametrize("bits", [0, 2, 9, -1])
def test_w_bits_range(bits):
    q, l = _w()
    with pytest.raises(ValueError, match="w_bits"):
        ext.dequant_kbit(q, l, bits)
    with pytest.raises(ValueError, match="w_bits"):
        ext.matmul_kbit(torch.zeros(1, 64, dtype=torch.float16), q, l, bits)


def test_w_bits_type():
    q, l = _w()
    with pytest.raises(TypeError):
        ext.dequant_kbit(q, l, 3.0)


def test_dtypes_and_dims():
    q, l = _w()
    with pytest.raises(ValueError, match="int32"):
        ext.dequant_kbit(q.to(torch.int64), l, 3)
    with pytest.raises(ValueError, match="3-D"):
        ext.dequant_kbit(q[0], l, 3)
    with pytest.raises(ValueError, match="float16"):
        ext.dequant_kbit(q, l.float(), 3)


def test_cpu_tensors_are_rejected_not_computed():
    q, l = _w()
    with pytest.raises(ValueError, match="GPU"):
        ext.dequant_kbit(q, l, 3)
    with pytest.raises(ValueError, match="GPU"):
        ext.matmul_kbit(torch.zeros(1, 64, dtype=torch.float16), q, l, 3)


def test_fused_gemm_dispatch_rule():
    """Where AnyPrecisionLinear takes the fused GEMM instead of dequant + matmul (the reference sends everything above
    8 rows to dequant + matmul, AnyPrecisionLinear.py:60-62): the rule as it was fitted to the measured sweep.  The
    thresholds live in the library (ap_gemm_kbit_pays); the module only asks."""
    from any_precision_amd.linear import fused_gemm_pays
    assert all(fused_gemm_pays(m, n, b, k) for m in (9, 32) for n in (4096, 14336) for b in (3, 8) for k in (4000, 4096))
    # rows the tiled kernel does not take (not a multiple of 128 elements): the K-split kernel's crossovers
    assert fused_gemm_pays(64, 4096, 8, 4000) and fused_gemm_pays(64, 14336, 5, 4000) and not fused_gemm_pays(64, 14336, 6, 4000)
    assert not fused_gemm_pays(65, 4096, 5, 8224) and not fused_gemm_pays(129, 4096, 6, 4000) and fused_gemm_pays(128, 4096, 6, 4000)
    assert not fused_gemm_pays(64, 14336, 8, 4000) and not fused_gemm_pays(200, 4096, 3, 4000)
    assert fused_gemm_pays(64, 1024, 8, 4096) and not fused_gemm_pays(64, 1024, 5, 8192)        # narrow, long rows
    # the tiled kernel, linears of at least 4096 rows: every bit-width up to 128 activation rows
    assert all(fused_gemm_pays(128, n, b, k) for b in (3, 8) for n, k in ((4096, 4096), (11008, 4096), (5120, 13824), (28672, 8192)))
    assert fused_gemm_pays(65, 14336, 8, 4096) and fused_gemm_pays(64, 5120, 8, 13824) and fused_gemm_pays(64, 8192, 8, 8192)
    # up to 256 at up to 5 bits; at 6 bits except beyond 16384 rows; at 7 and 8 bits on at most 8192 rows
    assert fused_gemm_pays(256, 11008, 4, 4096) and fused_gemm_pays(256, 28672, 5, 8192) and fused_gemm_pays(256, 13824, 6, 5120)
    assert not fused_gemm_pays(129, 28672, 6, 8192) and fused_gemm_pays(256, 8192, 8, 8192) and not fused_gemm_pays(257, 8192, 8, 8192)
    assert not fused_gemm_pays(129, 11008, 8, 4096) and fused_gemm_pays(256, 4096, 8, 4096) and fused_gemm_pays(256, 5120, 7, 13824)
    # up to 512 at 3 bits on at most 8192 rows
    assert fused_gemm_pays(512, 4096, 3, 11008) and fused_gemm_pays(512, 8192, 3, 8192) and not fused_gemm_pays(257, 11008, 3, 4096)
    assert not fused_gemm_pays(513, 4096, 3, 4096) and not fused_gemm_pays(257, 4096, 4, 4096)
    # linears of 1024..4095 rows: 3 and 4 bits up to 512
    assert fused_gemm_pays(100, 1024, 3, 4096) and fused_gemm_pays(512, 1024, 4, 8192) and not fused_gemm_pays(100, 1024, 5, 4096)
    assert not fused_gemm_pays(100, 512, 3, 4096)
    with pytest.raises(ValueError):
        fused_gemm_pays(16, 4096, 3, 4097)                # not a row length the layout has

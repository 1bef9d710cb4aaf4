"""The committed vectors of tests/golden/bitplane_small.npz against the oracle, the numpy
packer and (on a GPU) the HIP library.  The vectors are data only (codes, packed planes,
tables, expected fp16 weights and float64 GEMV results); tests/golden/make_vectors.py says
how they were made."""
import os

import numpy as np
import pytest

from _util import REL_TOL

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "bitplane_small.npz"), allow_pickle=False)
CASES = list(range(len(GOLD["shapes"])))


def _case(i):
    g = lambda k: GOLD[f"s{i}_{k}"]
    return g


@pytest.mark.parametrize("i", CASES)
def test_vectors_are_self_consistent(i):
    g = _case(i)
    N, K = GOLD["shapes"][i]
    assert g("codes").shape == (N, K) and g("qweight").shape == (8, N, K // 32) and g("qweight").dtype == np.int32
    for b in range(3, 9):
        want = np.take_along_axis(g(f"lut{b}"), (g("codes") >> (8 - b)).astype(np.int64), axis=1)
        assert np.array_equal(want.view(np.int16), g(f"w{b}").view(np.int16))
        np.testing.assert_allclose(g("x").astype(np.float64) @ want.astype(np.float64).T, g(f"y{b}"), rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("i", CASES)
def test_packers_reproduce_the_planes(i, oracle):
    from any_precision_amd.packing import pack_codes, unpack_codes
    g = _case(i)
    assert np.array_equal(pack_codes(g("codes"), 8), g("qweight"))
    assert np.array_equal(oracle.pack_bitplanes(g("codes"), 8), g("qweight"))
    assert np.array_equal(oracle.np_pack_bitplanes(g("codes"), 8), g("qweight"))
    assert np.array_equal(unpack_codes(g("qweight")), g("codes"))


@pytest.mark.parametrize("i", CASES)
def test_oracle_kernels_reproduce_the_results(i, oracle):
    g = _case(i)
    for b in range(3, 9):
        got = oracle.dequant_kbit(g("qweight"), g(f"lut{b}"), b)
        assert np.array_equal(got.view(np.int16), g(f"w{b}").view(np.int16)), b
        y16, y64 = oracle.matmul_kbit(g("x"), g("qweight"), g(f"lut{b}"), b, return_f64=True)
        np.testing.assert_allclose(y64, g(f"y{b}"), rtol=1e-11, atol=1e-11)
        assert np.array_equal(y16.view(np.int16), g(f"y{b}").astype(np.float16).view(np.int16)), b


@pytest.mark.gpu
@pytest.mark.parametrize("i", CASES)
def test_hip_library_reproduces_the_results(i):
    import torch
    import any_precision_ext as ext
    g = _case(i)
    q = torch.from_numpy(g("qweight")).cuda()
    x = torch.from_numpy(g("x")).cuda()
    for b in range(3, 9):
        print(f"golden case {i} b={b}", flush=True)
        lut = torch.from_numpy(g(f"lut{b}")).cuda()
        w = ext.dequant_kbit(q, lut, b).cpu().numpy()
        assert np.array_equal(w.view(np.int16), g(f"w{b}").view(np.int16)), b   # bit-exact
        want = g(f"y{b}")
        for fn in (ext.matmul_kbit, ext.gemm_kbit):
            y = fn(x, q, lut, b).float().cpu().numpy().astype(np.float64)
            # tolerance of the floating-point path: 1e-2 relative, normwise and against max |y|
            assert np.linalg.norm(y - want) <= REL_TOL * np.linalg.norm(want), (fn.__name__, b)
            assert np.abs(y - want).max() <= REL_TOL * np.abs(want).max(), (fn.__name__, b)

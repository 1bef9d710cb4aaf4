"""dequant_kbit on the GPU against the oracle: bit-exact, through the C ABI."""
import ctypes

import numpy as np
import pytest
import torch

from _util import assert_bit_exact, layer_to_gpu, make

pytestmark = pytest.mark.gpu

RAGGED = [(1, 32), (7, 32), (5, 96), (13, 1056), (4, 2080), (130, 992), (33, 1024), (3, 3104)]
FULL = [(4096, 4096), (11008, 4096), (4096, 11008), (1024, 4096), (4096, 14336)]


@pytest.fixture(scope="module")
def ext():
    import any_precision_ext
    return any_precision_ext


@pytest.mark.parametrize("N,K", RAGGED)
def test_ragged_shapes_all_bits(ext, oracle, N, K):
    L = make(N, K, seed=N + K)
    q, luts = layer_to_gpu(L)
    for b in range(3, 9):
        print(f"dequant N={N} K={K} b={b}", flush=True)
        got = ext.dequant_kbit(q, luts[b], b)
        assert got.shape == (N, K) and got.dtype == torch.float16
        assert_bit_exact(got, oracle.dequant_kbit(L.qweight, L.luts[b], b), f"N={N} K={K} b={b}")


@pytest.mark.parametrize("N,K", FULL)
def test_benchmark_shapes_all_bits(ext, oracle, N, K):
    L = make(N, K, seed=1)
    q, luts = layer_to_gpu(L)
    for b in range(3, 9):
        print(f"dequant N={N} K={K} b={b}", flush=True)
        got = ext.dequant_kbit(q, luts[b], b)
        want = np.take_along_axis(L.luts[b], (L.codes >> (8 - b)).astype(np.int64), axis=1)
        assert_bit_exact(got, want, f"N={N} K={K} b={b} (table lookup of top bits)")
        if b in (3, 8):
            assert_bit_exact(got, oracle.dequant_kbit(L.qweight, L.luts[b], b), f"N={N} K={K} b={b} (oracle)")


def test_pruned_planes_and_untouched_tail(ext, oracle):
    # prune_precisions keeps only the top planes; the kernel must not read beyond plane b-1.
    L = make(64, 2080, seed=9)
    for b in range(3, 9):
        q, luts = layer_to_gpu(L, planes=b)
        assert q.shape[0] == b
        assert_bit_exact(ext.dequant_kbit(q, luts[b], b), oracle.dequant_kbit(L.qweight, L.luts[b], b), f"b={b}")


def test_special_values_in_tables_are_copied_verbatim(ext, oracle):
    L = make(8, 1056, seed=2)
    lut = L.luts[4].copy().view(np.uint16)
    lut[:, 0] = 0x7C00      # +inf
    lut[:, 1] = 0x7E01      # a NaN payload
    lut[:, 2] = 0x8000      # -0
    lut[:, 3] = 0x0001      # smallest subnormal
    lut = lut.view(np.float16)
    q, _ = layer_to_gpu(L)
    got = ext.dequant_kbit(q, torch.from_numpy(lut).cuda(), 4)
    assert_bit_exact(got, oracle.dequant_kbit(L.qweight, lut, 4))


def test_non_default_stream_and_graph_replay(ext, oracle):
    L = make(256, 4096, seed=4)
    q, luts = layer_to_gpu(L)
    want = oracle.dequant_kbit(L.qweight, L.luts[5], 5)
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        got = ext.dequant_kbit(q, luts[5], 5)
    s.synchronize()
    assert_bit_exact(got, want, "side stream")

    from any_precision_amd import _capi
    out = torch.zeros((256, 4096), dtype=torch.float16, device="cuda")
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        rc = _capi.lib.ap_dequant_kbit(q.data_ptr(), luts[5].data_ptr(), out.data_ptr(), 256, 4096, 5,
                                       torch.cuda.current_stream().cuda_stream)
        assert rc == 0
    for rep in range(3):
        out.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert_bit_exact(out, want, f"graph replay {rep}")


def test_raw_c_abi_call(oracle):
    from any_precision_amd import _capi
    L = make(40, 1056, seed=6)
    q, luts = layer_to_gpu(L)
    out = torch.empty((40, 1056), dtype=torch.float16, device="cuda")
    rc = _capi.lib.ap_dequant_kbit(ctypes.c_void_p(q.data_ptr()), ctypes.c_void_p(luts[6].data_ptr()),
                                   ctypes.c_void_p(out.data_ptr()), 40, 1056, 6, None)
    assert rc == 0
    torch.cuda.synchronize()
    assert_bit_exact(out, oracle.dequant_kbit(L.qweight, L.luts[6], 6))


def test_idempotent_and_row_independent(ext):
    # size-independent properties at a full benchmark shape: same call twice is identical;
    # dequant of a row block equals the block of the full dequant.
    L = make(4096, 11008, seed=3)
    q, luts = layer_to_gpu(L)
    a = ext.dequant_kbit(q, luts[7], 7)
    b = ext.dequant_kbit(q, luts[7], 7)
    assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    sub = ext.dequant_kbit(q[:, 1000:1512].contiguous(), luts[7][1000:1512].contiguous(), 7)
    assert torch.equal(sub.view(torch.int16), a[1000:1512].view(torch.int16))

"""Seeded random sweep over shapes, bit-widths and batches: every op of the library against the
oracle (dequant bit-exact; GEMV / GEMM at 1e-2 relative), through the C ABI.  The shape
distribution favours the edges the kernels branch on: a handful of rows, row counts around
a workgroup boundary, rows of one to a few words, rows with a tail chunk, rows as long as the
benchmark shapes."""
import numpy as np
import pytest
import torch

from _util import assert_bit_exact, assert_close_gemv, layer_to_gpu, make
from any_precision_amd import synth

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_random_shapes(oracle, seed):
    import any_precision_ext as ext
    from any_precision_amd import _capi
    rng = np.random.default_rng(seed)
    rng2 = np.random.default_rng(seed + 100)
    for c in range(16):
        N = int(rng.choice([rng.integers(1, 70), rng.integers(70, 600), rng.integers(2040, 2100)]))
        words = int(rng.choice([rng.integers(1, 40), rng.integers(40, 400), rng.choice([128, 256, 344, 448])]))
        K = 32 * words
        N = min(N, max(1, int(4e6 // K)))
        b = int(rng.integers(3, 9))
        L = make(N, K, seed=1000 * seed + c)
        q, luts = layer_to_gpu(L)
        batches = (int(rng.integers(1, 9)), int(rng.integers(9, 129)))
        print(f"random case {seed}/{c}: N={N} K={K} b={b} M={batches}", flush=True)
        assert_bit_exact(ext.dequant_kbit(q, luts[b], b), oracle.dequant_kbit(L.qweight, L.luts[b], b),
                         f"N={N} K={K} b={b}")
        for M in batches:
            x = synth.make_x(M, K, seed=M + c)
            xg = torch.from_numpy(x).cuda()
            _, want = oracle.matmul_kbit(x, L.qweight, L.luts[b], b, return_f64=True)
            assert_close_gemv(ext.gemm_kbit(xg, q, luts[b], b), want, f"gemm N={N} K={K} b={b} M={M}")
            if M <= 8:
                assert_close_gemv(ext.matmul_kbit(xg, q, luts[b], b), want, f"matmul N={N} K={K} b={b} M={M}")
        if K % 128 == 0:
            # the tiled GEMM: forced with either tile and one or two K halves at the larger batch, and by the default
            # rule beyond 128 rows (its own generator, so that the cases above stay what they were)
            M = batches[1]
            tile, split = int(rng2.choice([4, 8])), int(rng2.choice([1, 2]))
            x = synth.make_x(M, K, seed=M + c)
            _, want = oracle.matmul_kbit(x, L.qweight, L.luts[b], b, return_f64=True)
            with _capi.tuning(gemm_tiled=2, gemm_tile=tile, gemm_tile_split=split):
                got = ext.gemm_kbit(torch.from_numpy(x).cuda(), q, luts[b], b)
            assert_close_gemv(got, want, f"tiled {tile}/{split} N={N} K={K} b={b} M={M}")
            if K >= 1024:   # tiles of 16 or 32 activation rows (what small grids take), case by case in turn
                with _capi.tuning(gemm_tiled=2, gemm_tile=1 + (c & 1)):
                    got = ext.gemm_kbit(torch.from_numpy(x).cuda(), q, luts[b], b)
                assert_close_gemv(got, want, f"tiled {1 + (c & 1)} N={N} K={K} b={b} M={M}")
            M = int(rng2.integers(129, 300))
            print(f"random case {seed}/{c}: tiled default M={M}", flush=True)
            x = synth.make_x(M, K, seed=M + c)
            _, want = oracle.matmul_kbit(x, L.qweight, L.luts[b], b, return_f64=True)
            assert_close_gemv(ext.gemm_kbit(torch.from_numpy(x).cuda(), q, luts[b], b), want, f"tiled N={N} K={K} b={b} M={M}")

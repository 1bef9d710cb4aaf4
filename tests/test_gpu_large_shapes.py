"""Largest shapes of the Llama family (70B MLP: 28672 x 8192 and 8192 x 28672) against a
reference written with torch ops on the GPU straight from the layout definition
(pack.py:51-68: element k of row n sits in word 32 c + t, byte group j, bit e with
k = 1024 c + 8 (32 j + t) + e) -- independent of the oracle and of the kernels' code, and big
enough to catch 32-bit overflow in the addressing."""
import pytest
import torch

from _util import REL_TOL

pytestmark = pytest.mark.gpu


def torch_indices(qweight, b):
    """int64 [N, K] index of every element from planes 0..b-1 (K a multiple of 1024)."""
    P, N, W = qweight.shape
    K = W * 32
    idx = torch.zeros((N, K), dtype=torch.int64, device=qweight.device)
    shifts = torch.arange(31, -1, -1, device=qweight.device, dtype=torch.int64)       # bit of (j, e), MSB first
    for p in range(b):
        words = qweight[p].to(torch.int64) & 0xFFFFFFFF                              # [N, W]
        bits = (words.unsqueeze(-1) >> shifts) & 1                                    # [N, W, (j e)]
        bits = bits.view(N, K // 1024, 32, 4, 8).permute(0, 1, 3, 2, 4).reshape(N, K)  # [n, c, j, t, e]
        idx |= bits << (b - 1 - p)
        del words, bits
    return idx


@pytest.mark.parametrize("N,K", [(28672, 8192), (8192, 28672)])
def test_llama70b_mlp_shapes(N, K):
    import any_precision_ext as ext
    gen = torch.Generator(device="cuda")
    gen.manual_seed(N)
    q = torch.randint(-2**31, 2**31 - 1, (8, N, K // 32), dtype=torch.int32, device="cuda", generator=gen)
    for b in (3, 8):
        print(f"large N={N} K={K} b={b}", flush=True)
        lut = torch.sort(torch.randn((N, 1 << b), device="cuda", generator=gen) * 0.02, dim=1).values.half()
        want_w = torch.gather(lut, 1, torch_indices(q, b))
        got_w = ext.dequant_kbit(q, lut, b)
        assert torch.equal(got_w, want_w), f"dequant N={N} K={K} b={b}"
        del got_w
        # 200 and 520 rows: the tiled GEMM (tiles of 64 x 128 rows here, four and five of them along the activation rows)
        for M, fn in ((1, ext.matmul_kbit), (4, ext.matmul_kbit), (8, ext.matmul_kbit), (32, ext.gemm_kbit), (200, ext.gemm_kbit),
                      (520, ext.gemm_kbit)):
            x = torch.randn((M, K), device="cuda", generator=gen).half()
            want = x.double() @ want_w.double().T
            got = fn(x, q, lut, b).double()
            assert (got - want).norm() <= REL_TOL * want.norm(), f"{fn.__name__} M={M} b={b}"
            assert (got - want).abs().max() <= REL_TOL * want.abs().max(), f"{fn.__name__} M={M} b={b}"
        del want_w


def test_llama3_8b_mlp_shape_under_the_default_routing():
    """14336 x 4096 at M = 1..8 under the default routing: the dot-product kernel (1, 2 and part of
    3), the 4x4x4 matrix-core kernel with one (3, 4) and two (5..8) groups of activation rows; then the
    fused GEMM at 16, 32 and 48 rows (K-split kernel up to 32, tiled kernel beyond) and at 100 and 300."""
    import any_precision_ext as ext
    N, K = 14336, 4096
    gen = torch.Generator(device="cuda")
    gen.manual_seed(5)
    q = torch.randint(-2**31, 2**31 - 1, (8, N, K // 32), dtype=torch.int32, device="cuda", generator=gen)
    for b in (3, 4, 5, 6, 7, 8):
        lut = torch.sort(torch.randn((N, 1 << b), device="cuda", generator=gen) * 0.02, dim=1).values.half()
        want_w = torch.gather(lut, 1, torch_indices(q, b)).double()
        for M in range(1, 9):
            print(f"llama3 mlp b={b} M={M}", flush=True)
            x = torch.randn((M, K), device="cuda", generator=gen).half()
            want = x.double() @ want_w.T
            got = ext.matmul_kbit(x, q, lut, b).double()
            assert (got - want).norm() <= REL_TOL * want.norm(), f"M={M} b={b}"
            assert (got - want).abs().max() <= REL_TOL * want.abs().max(), f"M={M} b={b}"
        # the fused GEMM under its default routing: two weight-row blocks per workgroup at up to 5 / 6
        # bits, chunks of 32 activation rows above 32
        for M in (16, 32, 48, 100, 300):
            print(f"llama3 mlp gemm b={b} M={M}", flush=True)
            x = torch.randn((M, K), device="cuda", generator=gen).half()
            want = x.double() @ want_w.T
            got = ext.gemm_kbit(x, q, lut, b).double()
            assert (got - want).norm() <= REL_TOL * want.norm(), f"gemm M={M} b={b}"
            assert (got - want).abs().max() <= REL_TOL * want.abs().max(), f"gemm M={M} b={b}"
        del want_w


@pytest.mark.parametrize("N,K", [(2560, 2560), (10240, 2560), (2560, 10240)])
def test_phi2_shapes_against_the_oracle(N, K, oracle):
    """Linear shapes of Phi-2 (hidden 2560: rows of 2.5 chunks, tail chunk of 16 words; the reference's
    analyzer/architectures/phi.yaml lists the model) through every op, against the oracle."""
    import numpy as np
    import any_precision_ext as ext
    from _util import assert_bit_exact, assert_close_gemv, layer_to_gpu, make
    from any_precision_amd import synth
    L = make(N, K, seed=N // 10 + K)
    q, luts = layer_to_gpu(L)
    for b in (3, 5, 8):
        print(f"phi2 N={N} K={K} b={b}", flush=True)
        want_w = np.take_along_axis(L.luts[b], (L.codes >> (8 - b)).astype(np.int64), axis=1)
        assert_bit_exact(ext.dequant_kbit(q, luts[b], b), want_w, f"dequant N={N} K={K} b={b}")
        for M, fn in ((1, ext.matmul_kbit), (4, ext.matmul_kbit), (8, ext.matmul_kbit), (16, ext.gemm_kbit)):
            x = synth.make_x(M, K, seed=M)
            _, want = oracle.matmul_kbit(x, L.qweight, L.luts[b], b, return_f64=True)
            assert_close_gemv(fn(torch.from_numpy(x).cuda(), q, luts[b], b), want, f"{fn.__name__} N={N} K={K} b={b} M={M}")

"""Batch 32 x 512-token prefill: 16384 activation rows through one linear, on the three Llama-2-7B shapes.

Two routes compute ``x @ dequant(qweight, lut, b).T`` (the reference's branch for more than 8 rows,
any_precision/modules/AnyPrecisionLinear.py:60-62): the module's forward (``dequant_kbit`` + library GEMM at this
size) and ``gemm_kbit`` (the fused tiled kernel, here with tiles of 128 activation rows and 128 tiles along the
rows, the order of tiles that grids of more than 8 row tiles take).  Both are checked against the oracle on a
slice (128 weight rows x 256 sampled activation rows) and against each other over the whole [16384, N] result.
Tolerance: 1e-2 relative, normwise and against the largest magnitude (fp32 accumulate, fp16 out).
"""
import numpy as np
import pytest
import torch

from _util import REL_TOL, assert_close_gemv

pytestmark = pytest.mark.gpu

PREFILL_ROWS = 32 * 512


@pytest.mark.parametrize("N,K", [(4096, 4096), (11008, 4096), (4096, 11008)])
def test_prefill_16384_rows_module_and_fused_gemm(N, K, oracle):
    import any_precision_ext as ext
    from any_precision_amd import AnyPrecisionLinear, synth
    from any_precision_amd.packing import pack_codes

    rng = np.random.default_rng(N + K)
    # oracle-checked slice: 128 consecutive weight rows (two tiles of 64, not aligned to a tile of 128) get seeded
    # codes and tables from numpy; the other rows come from the GPU generator
    r0 = 64 * 5
    rows = slice(r0, r0 + 128)
    codes = rng.integers(0, 256, size=(128, K), dtype=np.uint8)
    planes_slice = pack_codes(codes, 8)                                   # int32 [8, 128, K/32]
    gen = torch.Generator(device="cuda")
    gen.manual_seed(N * 7 + K)
    q = torch.randint(-2**31, 2**31 - 1, (8, N, K // 32), dtype=torch.int32, device="cuda", generator=gen)
    q[:, rows] = torch.from_numpy(planes_slice).cuda()
    x = torch.randn((32, 512, K), device="cuda", generator=gen).half()    # batch 32 x 512 tokens
    pick = np.sort(rng.choice(PREFILL_ROWS, size=256, replace=False))
    pick[0], pick[-1] = 0, PREFILL_ROWS - 1                               # first and last row of the batch too
    x_pick = x.view(PREFILL_ROWS, K)[torch.from_numpy(pick).cuda()].cpu().numpy()

    for b in (3, 8):
        print(f"prefill N={N} K={K} b={b}", flush=True)
        table = torch.sort(torch.randn((N, 1 << b), device="cuda", generator=gen) * 0.02, dim=1).values.half()
        table_slice = table[rows].cpu().numpy()
        _, want = oracle.matmul_kbit(x_pick, planes_slice, table_slice, b, return_f64=True)   # [256, 128]

        lin = AnyPrecisionLinear(K, N, [b], bias=False, device="cuda")
        lin.qweight = q[:b]
        lin._buffers[f"lut{b}"] = table
        y_mod = lin(x, precision=b)
        assert y_mod.shape == (32, 512, N) and y_mod.dtype == torch.float16
        y_fused = ext.gemm_kbit(x, q, table, b)
        assert y_fused.shape == (32, 512, N)
        torch.cuda.synchronize()

        sel = torch.from_numpy(pick).cuda()
        for name, y in (("module", y_mod), ("gemm_kbit", y_fused)):
            got = y.view(PREFILL_ROWS, N)[sel][:, rows]
            assert_close_gemv(got, want, f"{name} N={N} K={K} b={b} vs oracle")
        # the two routes over the whole result (chunks of rows keep the fp32 temporaries small)
        a, c = y_mod.view(PREFILL_ROWS, N), y_fused.view(PREFILL_ROWS, N)
        num = den = 0.0
        worst = top = 0.0
        for m0 in range(0, PREFILL_ROWS, 2048):
            fa, fc = a[m0:m0 + 2048].float(), c[m0:m0 + 2048].float()
            assert torch.isfinite(fa).all() and torch.isfinite(fc).all()
            num += float((fa - fc).double().pow(2).sum())
            den += float(fa.double().pow(2).sum())
            worst = max(worst, float((fa - fc).abs().max()))
            top = max(top, float(fa.abs().max()))
        assert num ** 0.5 <= REL_TOL * den ** 0.5, f"module vs gemm_kbit N={N} K={K} b={b}: {num ** 0.5 / den ** 0.5:.3e}"
        assert worst <= REL_TOL * top, f"module vs gemm_kbit N={N} K={K} b={b}: max abs {worst:.3e} of {top:.3e}"
        del y_mod, y_fused, lin, table

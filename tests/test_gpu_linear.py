"""AnyPrecisionLinear on the GPU: state-dict format, precision switching, both batch branches."""
import numpy as np
import pytest
import torch

from _util import assert_close_gemv, make
from any_precision_amd import packing, synth

pytestmark = pytest.mark.gpu


def _module(L, bias=True, precisions=None):
    from any_precision_amd import AnyPrecisionLinear
    bits = list(range(L.seed_bits, L.parent_bits + 1))
    m = AnyPrecisionLinear(L.K, L.N, bits, bias=bias, precisions=precisions, device="cuda", dtype=torch.float16)
    sd = {k: torch.from_numpy(v) for k, v in packing.pack_layer(L.codes, L.luts).items()}
    if bias:
        sd["bias"] = torch.from_numpy(np.linspace(-1, 1, L.N).astype(np.float16))
    m.load_state_dict(sd)
    return m, sd


def test_state_dict_keys_shapes_dtypes():
    L = make(64, 1056, seed=0)
    m, _ = _module(L)
    sd = m.state_dict()
    assert sorted(sd) == sorted(["qweight", "bias"] + [f"lut{b}" for b in range(3, 9)])
    assert sd["qweight"].shape == (8, 64, 33) and sd["qweight"].dtype == torch.int32
    for b in range(3, 9):
        assert sd[f"lut{b}"].shape == (64, 1 << b) and sd[f"lut{b}"].dtype == torch.float16
    assert m.precision == 8 and m.precisions == list(range(3, 9))


def test_forward_every_branch_and_bias(oracle):
    L = make(128, 4096, seed=1)
    m, sd = _module(L)
    bias = sd["bias"].numpy().astype(np.float64)
    for b in (3, 5, 8):
        for M in (1, 8, 9, 32, 33, 64, 65, 128, 130): # GEMV | fused GEMM (to 128 rows here: 128 x 4096) | dequant + matmul
            x = synth.make_x(M, L.K, seed=M)
            y = m(torch.from_numpy(x).cuda(), precision=b)
            _, want = oracle.matmul_kbit(x, L.qweight, L.luts[b], b, return_f64=True)
            assert y.shape == (M, L.N)
            assert_close_gemv(y, want + bias, f"b={b} M={M}")


def test_strided_activations_are_accepted_on_every_branch(oracle):
    """A transposed or sliced activation view (as Hugging Face modules hand over now and then) gives the
    result of its dense copy on the GEMV, the fused-GEMM and the dequant + matmul branch alike."""
    L = make(96, 2048, seed=4)
    m, sd = _module(L, bias=False)
    for M in (1, 4, 8, 20, 70):
        x = synth.make_x(M, 2 * L.K, seed=M)
        xg = torch.from_numpy(x).cuda()[:, ::2]                 # every other column: stride 2
        assert not xg.is_contiguous()
        _, want = oracle.matmul_kbit(np.ascontiguousarray(x[:, ::2]), L.qweight, L.luts[4], 4, return_f64=True)
        assert_close_gemv(m(xg, precision=4), want, f"strided M={M}")
        xt = torch.from_numpy(np.ascontiguousarray(x[:, ::2].T)).cuda().T    # transposed view of a [K, M] tensor
        assert not xt.is_contiguous() or M == 1
        assert_close_gemv(m(xt, precision=4), want, f"transposed M={M}")


def test_set_precision_and_prune(oracle):
    L = make(32, 1024, seed=2)
    m, _ = _module(L, bias=False, precisions=[3, 4, 6])
    assert m.precision == 6
    with pytest.raises(RuntimeError):
        m.set_precision(8)
    m.prune_precisions()
    assert m.qweight.shape[0] == 6
    assert not hasattr(m, "lut8") and not hasattr(m, "lut5") and hasattr(m, "lut4")
    x = synth.make_x(2, L.K)
    for b in (3, 4, 6):
        m.set_precision(b)
        _, want = oracle.matmul_kbit(x, L.qweight, L.luts[b], b, return_f64=True)
        assert_close_gemv(m(torch.from_numpy(x).cuda()), want, f"b={b}")


def test_constructor_errors():
    from any_precision_amd import AnyPrecisionLinear
    with pytest.raises(RuntimeError):
        AnyPrecisionLinear(64, 8, [3, 4], dtype=torch.float32)
    with pytest.raises(RuntimeError):
        AnyPrecisionLinear(64, 8, [3, 4], precisions=(3, 4))


def test_forward_group_equals_module_by_module(oracle):
    """forward_group (one launch where the dot-product kernel serves the set, a launch per member otherwise, module
    by module beyond 8 rows) against the modules called one by one: the oracle's values at the path's bar, with
    and without biases, joined or as a list."""
    from any_precision_amd.linear import forward_group, forward_swiglu
    layers = [make(n, 4096, seed=70 + n) for n in (256, 64, 64)]
    for bias in (False, True):
        mods = [_module(L, bias=bias)[0] for L in layers]
        for b in (3, 8):
            for rows in (1, 3, 6, 8, 9):
                print(f"forward_group bias={bias} b={b} rows={rows}", flush=True)
                x = synth.make_x(rows, 4096, seed=rows)
                xg = torch.from_numpy(x).cuda()
                outs = forward_group(mods, xg, b)
                joined = forward_group(mods, xg, b, concat=True)
                assert joined.shape == (rows, 384) and torch.equal(joined, torch.cat(outs, dim=-1))
                for L, m, got in zip(layers, mods, outs):
                    _, want = oracle.matmul_kbit(x, L.qweight, L.luts[b], b, return_f64=True)
                    if bias:
                        want = want + m.bias.double().cpu().numpy()
                    assert_close_gemv(got, want, f"forward_group bias={bias} b={b} rows={rows} N={L.N}")
    # SiLU(gate) * up through the one-launch form (up to 4 rows) and through its fallback
    gate, up = _module(layers[1], bias=False)[0], _module(layers[2], bias=False)[0]
    for rows in (2, 6):
        xg = torch.from_numpy(synth.make_x(rows, 4096, seed=9)).cuda()
        got = forward_swiglu(gate, up, xg, 4)
        want = torch.nn.functional.silu(gate(xg, precision=4).float()) * up(xg, precision=4).float()
        assert (got.float() - want).abs().max().item() <= 1e-2 * want.abs().max().item()


def test_forward_takes_the_tiled_gemm_up_to_256_rows_at_3_and_4_bits(oracle):
    """A linear of 4096 rows of a multiple of 128 elements: up to 6 bits go through the fused GEMM up to 256 activation
    rows (3 bits up to 512), 6 bits beyond 256 rows and anything beyond 512 through dequant + matmul; all against the
    oracle."""
    from any_precision_amd.linear import fused_gemm_pays
    L = make(4096, 256, seed=5)
    m, _ = _module(L, bias=False)
    assert fused_gemm_pays(200, 4096, 3, 256) and fused_gemm_pays(256, 4096, 4, 256)
    assert fused_gemm_pays(200, 4096, 5, 256) and fused_gemm_pays(200, 4096, 6, 256) and not fused_gemm_pays(257, 4096, 6, 256)
    assert fused_gemm_pays(257, 4096, 3, 256) and not fused_gemm_pays(513, 4096, 3, 256)
    for b, M in ((3, 200), (3, 256), (4, 256), (5, 200), (6, 200), (6, 257), (8, 256), (3, 257), (3, 513)):
        print(f"linear tiled b={b} M={M}", flush=True)
        x = synth.make_x(M, L.K, seed=M)
        y = m(torch.from_numpy(x).cuda(), precision=b)
        _, want = oracle.matmul_kbit(x, L.qweight, L.luts[b], b, return_f64=True)
        assert_close_gemv(y, want, f"b={b} M={M}")


def test_forward_group_beyond_32_rows_is_one_tiled_launch(oracle):
    """Sets of linears on 9..256 rows go through gemm_kbit_group (one launch of the tiled kernel) where fused_set_pays
    says so, with biases added afterwards; against the oracle, joined or as a list."""
    from any_precision_amd.linear import forward_group, fused_set_pays
    assert fused_set_pays(128, [4096, 4096, 4096], 3, 4096) and fused_set_pays(256, [11008, 11008], 5, 4096)
    assert fused_set_pays(128, [11008, 11008], 8, 4096) and not fused_set_pays(129, [11008, 11008], 8, 4096)
    assert fused_set_pays(256, [4096, 4096, 4096], 8, 4096)
    assert fused_set_pays(128, [4096, 1024, 1024], 8, 4096) and fused_set_pays(9, [4096, 4096], 3, 4096)
    assert not fused_set_pays(32, [11008, 11008], 3, 4096) and not fused_set_pays(8, [4096, 4096], 3, 4096)
    assert fused_set_pays(16, [8192, 1024, 1024], 8, 8192) and not fused_set_pays(16, [8192, 8200], 8, 8192)
    assert fused_set_pays(257, [4096, 4096], 3, 4096) and not fused_set_pays(257, [4096, 4096], 4, 4096)
    assert not fused_set_pays(513, [4096, 4096], 3, 4096) and not fused_set_pays(300, [11008, 11008], 3, 4096)
    assert not fused_set_pays(64, [4096, 4096], 3, 4000)
    layers = [make(n, 256, seed=80 + n) for n in (4096, 512, 520)]
    for bias in (False, True):
        mods = [_module(L, bias=bias)[0] for L in layers]
        for b, rows in ((3, 40), (8, 64), (5, 200), (8, 200), (3, 300)):
            print(f"forward_group tiled bias={bias} b={b} rows={rows}", flush=True)
            x = synth.make_x(rows, 256, seed=rows)
            xg = torch.from_numpy(x).cuda()
            outs = forward_group(mods, xg, b)
            joined = forward_group(mods, xg, b, concat=True)
            assert joined.shape == (rows, 5128) and torch.equal(joined, torch.cat(outs, dim=-1))
            for L, m, got in zip(layers, mods, outs):
                _, want = oracle.matmul_kbit(x, L.qweight, L.luts[b], b, return_f64=True)
                if bias:
                    want = want + m.bias.double().cpu().numpy()
                assert_close_gemv(got, want, f"forward_group tiled bias={bias} b={b} rows={rows} N={L.N}")
    # 9..32 rows: sets whose members all have fewer than 8192 rows of at least 1024 elements (tiles of 16 or 32 rows)
    layers = [make(n, 1024, seed=90 + n) for n in (4096, 200)]
    mods = [_module(L, bias=False)[0] for L in layers]
    for b, rows in ((3, 12), (6, 20), (8, 32)):
        print(f"forward_group narrow tiles b={b} rows={rows}", flush=True)
        x = synth.make_x(rows, 1024, seed=rows)
        outs = forward_group(mods, torch.from_numpy(x).cuda(), b)
        for L, got in zip(layers, outs):
            _, want = oracle.matmul_kbit(x, L.qweight, L.luts[b], b, return_f64=True)
            assert_close_gemv(got, want, f"forward_group narrow tiles b={b} rows={rows} N={L.N}")

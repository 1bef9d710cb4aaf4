"""matmul_kbit on the GPU against the oracle, through the C ABI.

Tolerance: 1e-2 relative (normwise and against max |y|), fp32 accumulate / fp16 out
on the GPU against double accumulate / one rounding in the oracle."""
import numpy as np
import pytest
import torch

from _util import assert_bit_exact, assert_close_gemv, layer_to_gpu, make
from any_precision_amd import synth

pytestmark = pytest.mark.gpu

RAGGED = [(1, 32), (7, 32), (5, 96), (13, 1056), (4, 2080), (130, 992), (33, 1024), (3, 3104), (21, 4128)]
FULL = [(4096, 4096), (11008, 4096), (4096, 11008), (1024, 4096), (14336, 4096), (4096, 14336)]
SLICES = [(256, 4096), (192, 11008), (160, 14336)]


@pytest.fixture(scope="module")
def ext():
    import any_precision_ext
    return any_precision_ext


def _x(M, K, seed=0):
    x = synth.make_x(M, K, seed)
    return x, torch.from_numpy(x).cuda()


@pytest.mark.parametrize("N,K", RAGGED)
def test_ragged_shapes_all_bits_all_batches(ext, oracle, N, K):
    L = make(N, K, seed=N + K)
    q, luts = layer_to_gpu(L)
    for b in range(3, 9):
        for M in range(1, 9):
            print(f"gemv N={N} K={K} b={b} M={M}", flush=True)
            x, xg = _x(M, K, seed=M)
            got = ext.matmul_kbit(xg, q, luts[b], b)
            assert got.shape == (M, N) and got.dtype == torch.float16
            _, want = oracle.matmul_kbit(x, L.qweight, L.luts[b], b, return_f64=True)
            assert_close_gemv(got, want, f"N={N} K={K} b={b} M={M}")


@pytest.mark.parametrize("N,K", SLICES)
def test_row_slices_of_benchmark_shapes_all_batches(ext, oracle, N, K):
    L = make(N, K, seed=5)
    q, luts = layer_to_gpu(L)
    for b in range(3, 9):
        for M in range(1, 9):
            print(f"gemv N={N} K={K} b={b} M={M}", flush=True)
            x, xg = _x(M, K, seed=M)
            got = ext.matmul_kbit(xg, q, luts[b], b)
            _, want = oracle.matmul_kbit(x, L.qweight, L.luts[b], b, return_f64=True)
            assert_close_gemv(got, want, f"N={N} K={K} b={b} M={M}")


@pytest.mark.parametrize("N,K", FULL)
def test_benchmark_shapes(ext, oracle, N, K):
    L = make(N, K, seed=1)
    q, luts = layer_to_gpu(L)
    for b in range(3, 9):
        for M in (1, 8):
            print(f"gemv N={N} K={K} b={b} M={M}", flush=True)
            x, xg = _x(M, K, seed=M)
            got = ext.matmul_kbit(xg, q, luts[b], b)
            _, want = oracle.matmul_kbit(x, L.qweight, L.luts[b], b, return_f64=True)
            assert_close_gemv(got, want, f"N={N} K={K} b={b} M={M}")


def test_one_hot_x_returns_dequant_column_exactly(ext, oracle):
    # with a single 1.0 in x the sum has one non-zero term: the result is the table entry itself
    N, K = 96, 3104
    L = make(N, K, seed=8)
    q, luts = layer_to_gpu(L)
    for b in (3, 4, 6, 8):
        w = oracle.dequant_kbit(L.qweight, L.luts[b], b)
        for k in (0, 7, 8, 255, 256, 1023, 1024, 2047, 2048, 3071, 3072, 3080, 3103):
            x = torch.zeros((1, K), dtype=torch.float16, device="cuda")
            x[0, k] = 1.0
            got = ext.matmul_kbit(x, q, luts[b], b)
            assert_bit_exact(got[0], w[:, k], f"b={b} k={k}")


def test_constant_table_gives_scaled_sum(ext):
    N, K = 64, 11008
    L = make(N, K, seed=2)
    q, _ = layer_to_gpu(L)
    x, xg = _x(2, K)
    lut = torch.full((N, 32), 0.5, dtype=torch.float16, device="cuda")
    got = ext.matmul_kbit(xg, q, lut, 5)
    want = 0.5 * x.astype(np.float64).sum(axis=1, keepdims=True) * np.ones((1, N))
    assert_close_gemv(got, want, "constant table")


def test_leading_dims_and_determinism(ext, oracle):
    N, K = 512, 4096
    L = make(N, K, seed=3)
    q, luts = layer_to_gpu(L)
    x = synth.make_x(6, K).reshape(2, 3, K)
    xg = torch.from_numpy(x).cuda()
    a = ext.matmul_kbit(xg, q, luts[6], 6)
    assert a.shape == (2, 3, N)
    b = ext.matmul_kbit(xg.reshape(6, K), q, luts[6], 6)
    assert torch.equal(a.reshape(6, N).view(torch.int16), b.view(torch.int16))
    for _ in range(3):
        assert torch.equal(ext.matmul_kbit(xg, q, luts[6], 6).view(torch.int16), a.view(torch.int16))
    v = ext.matmul_kbit(xg[0, 0], q, luts[6], 6)      # 1-D input, as the reference allows
    assert v.shape == (N,)


def test_pruned_planes(ext, oracle):
    L = make(64, 4096, seed=9)
    x, xg = _x(1, 4096)
    for b in range(3, 9):
        q, luts = layer_to_gpu(L, planes=b)
        _, want = oracle.matmul_kbit(x, L.qweight, L.luts[b], b, return_f64=True)
        assert_close_gemv(ext.matmul_kbit(xg, q, luts[b], b), want, f"b={b}")


def test_batch_above_8_is_rejected_like_the_reference_assert(ext):
    L = make(8, 64, seed=0)
    q, luts = layer_to_gpu(L)
    with pytest.raises(ValueError, match="1..8"):
        ext.matmul_kbit(torch.zeros((9, 64), dtype=torch.float16, device="cuda"), q, luts[3], 3)
    with pytest.raises(ValueError, match="planes"):
        ext.matmul_kbit(torch.zeros((1, 64), dtype=torch.float16, device="cuda"), q[:3].contiguous(), luts[4], 4)
    with pytest.raises(ValueError, match="contiguous"):
        ext.matmul_kbit(torch.zeros((1, 128), dtype=torch.float16, device="cuda")[:, ::2], q, luts[3], 3)


def test_graph_replay_matches_eager(ext):
    from any_precision_amd import _capi
    N, K = 1024, 4096
    L = make(N, K, seed=4)
    q, luts = layer_to_gpu(L)
    _, xg = _x(1, K)
    eager = ext.matmul_kbit(xg, q, luts[4], 4)
    out = torch.zeros((1, N), dtype=torch.float16, device="cuda")
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        rc = _capi.lib.ap_matmul_kbit(xg.data_ptr(), q.data_ptr(), luts[4].data_ptr(), out.data_ptr(), 1, N, K, 4,
                                      torch.cuda.current_stream().cuda_stream)
        assert rc == 0
    for rep in range(3):
        out.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), eager.view(torch.int16)), rep


@pytest.mark.parametrize("K,Ns", [(4096, (512, 128, 128)), (1056, (33, 7, 64, 5)), (11008, (96, 96)), (96, (3,))])
def test_group_launch_equals_separate_calls_bit_for_bit(ext, oracle, K, Ns):
    """One launch for several linears: the same bits as one call per linear while the same kernel serves
    both (the alternative dot-product kernels, which only single calls use, switched off), and the oracle's
    values at the path's bar either way."""
    from any_precision_amd import _capi
    layers = [make(N, K, seed=40 + i) for i, N in enumerate(Ns)]
    gpu = [layer_to_gpu(L) for L in layers]
    for b in (3, 4, 5, 8):
        for M in (1, 2, 3, 4, 6):      # 6: the members go through the MFMA kernel one by one
            print(f"group K={K} Ns={Ns} b={b} M={M}", flush=True)
            x, xg = _x(M, K, seed=M)
            outs = ext.matmul_kbit_group(xg, [q for q, _ in gpu], [luts[b] for _, luts in gpu], b)
            assert len(outs) == len(Ns)
            for (q, luts), L, got in zip(gpu, layers, outs):
                assert got.shape == (M, L.N)
                with _capi.tuning(gemv_stream=0, gemv_fine=0):
                    single = ext.matmul_kbit(xg, q, luts[b], b)
                assert torch.equal(got, single)
                _, want = oracle.matmul_kbit(x, L.qweight, L.luts[b], b, return_f64=True)
                assert_close_gemv(got, want, f"K={K} N={L.N} b={b} M={M}")
                assert_close_gemv(ext.matmul_kbit(xg, q, luts[b], b), want, f"single K={K} N={L.N} b={b} M={M}")


def test_group_argument_errors(ext):
    L = make(8, 64, seed=0)
    q, luts = layer_to_gpu(L)
    _, xg = _x(1, 64)
    with pytest.raises(ValueError):
        ext.matmul_kbit_group(xg, [q] * 5, [luts[3]] * 5, 3)          # more members than a launch holds
    with pytest.raises(ValueError):
        ext.matmul_kbit_group(xg, [q, q], [luts[3]], 3)
    L2 = make(8, 96, seed=1)
    q2, luts2 = layer_to_gpu(L2)
    with pytest.raises(ValueError):
        ext.matmul_kbit_group(xg, [q, q2], [luts[3], luts2[3]], 3)    # different in_features


def test_every_kernel_for_small_batches_agrees_with_the_oracle(ext, oracle):
    """ap_matmul_kbit picks between the dot-product kernel, the 4x4x4 and the 16x16x32 matrix-core kernels by shape,
    rows and bit-width; the tuning knobs force each (matmul_mfma4: 0 never, 2 wherever it fits; matmul_mfma_from:
    the row count from which the 16x16x32 kernel runs, 9 = never), so each is run on shapes the default rule
    would give to another."""
    from any_precision_amd import _capi
    for N, K in ((40, 2080), (2056, 1024), (9, 11008)):
        L = make(N, K, seed=N)
        q, luts = layer_to_gpu(L)
        for b in (3, 6, 8):
            for M in (2, 3, 4, 5, 7, 8):
                x, xg = _x(M, K, seed=M)
                _, want = oracle.matmul_kbit(x, L.qweight, L.luts[b], b, return_f64=True)
                for mode in (0, 2):
                    print(f"forced kernel mfma4={mode} N={N} K={K} b={b} M={M}", flush=True)
                    with _capi.tuning(matmul_mfma4=mode):
                        got = ext.matmul_kbit(xg, q, luts[b], b)
                    assert_close_gemv(got, want, f"mfma4={mode} N={N} K={K} b={b} M={M}")
                for start, route in ((2, "mfma16"), (9, "dot")):
                    print(f"forced kernel mfma_from={start} N={N} K={K} b={b} M={M}", flush=True)
                    with _capi.tuning(matmul_mfma4=0, matmul_mfma_from=start, gemv_stream=0, gemv_fine=0):
                        assert _capi.matmul_route(M, N, K, b) == route
                        got = ext.matmul_kbit(xg, q, luts[b], b)
                    assert_close_gemv(got, want, f"mfma_from={start} N={N} K={K} b={b} M={M}")


# (rows, elements per row): tails (K % 1024 != 0), one word group, one/several waves per row, many rows
WAVE_SPLIT_SHAPES = [(2, 64), (130, 128), (34, 1088), (10, 2048), (64, 4096), (256, 11008), (20, 8192), (12, 14336),
                     (6, 28672), (1030, 1024)]


@pytest.mark.parametrize("knob", ["gemv_fine", "gemv_stream"])
def test_the_other_splits_of_the_work_over_waves_agree_with_the_oracle(ext, oracle, knob):
    """Two more dot-product kernels serve 1..4 activation rows (fine-grained row pairs, row-streaming
    row pairs with 16-byte loads); the default rule uses them on a few wide shapes
    only, so each is forced (knob = 2) over ragged and tail shapes, every bit-width, M = 1..4, and checked
    against the oracle at the path's 1e-2 bar.  Shapes a kernel does not serve (odd row counts, rows that
    are not a multiple of 64 / 128 elements) must fall through to the default kernels."""
    from any_precision_amd import _capi
    for N, K in WAVE_SPLIT_SHAPES + [(7, 4096), (5, 96), (4, 2080)]:
        L = make(N, K, seed=N + K)
        q, luts = layer_to_gpu(L)
        for b in range(3, 9):
            for M in (1, 2, 3, 4):
                print(f"{knob} N={N} K={K} b={b} M={M}", flush=True)
                x, xg = _x(M, K, seed=M)
                _, want = oracle.matmul_kbit(x, L.qweight, L.luts[b], b, return_f64=True)
                for waves in ((1, 24) if knob != "gemv_fine" else (0,)):
                    extra = {knob + "_waves": waves} if waves else {}
                    with _capi.tuning(**{knob: 2}, **extra):
                        got = ext.matmul_kbit(xg, q, luts[b], b)
                    assert_close_gemv(got, want, f"{knob} waves={waves} N={N} K={K} b={b} M={M}")


@pytest.mark.parametrize("knob", ["gemv_fine", "gemv_stream"])
def test_the_other_splits_are_exact_on_one_hot_activations_and_deterministic(ext, oracle, knob):
    """x = e_k picks column k of the dequantised weight: the fp16 result must be that table entry bit for
    bit (covers the word -> element mapping of every lane, tail chunk included); two runs must agree."""
    from any_precision_amd import _capi
    N, K = 66, 11008
    L = make(N, K, seed=5)
    q, luts = layer_to_gpu(L)
    for b in (3, 4, 5, 8):
        w = oracle.dequant_kbit(L.qweight, L.luts[b], b)
        for k in (0, 7, 8, 255, 256, 1023, 1024, 4095, 4096, 10239, 10240, 10431, 10432, 11007):
            x = np.zeros((1, K), dtype=np.float16)
            x[0, k] = 1.0
            with _capi.tuning(**{knob: 2}):
                got = ext.matmul_kbit(torch.from_numpy(x).cuda(), q, luts[b], b)
            assert_bit_exact(got, w[:, k].reshape(1, N), f"{knob} b={b} k={k}")
        x, xg = _x(3, K, seed=b)
        with _capi.tuning(**{knob: 2}):
            first = ext.matmul_kbit(xg, q, luts[b], b)
            again = ext.matmul_kbit(xg, q, luts[b], b)
        assert torch.equal(first.view(torch.int16), again.view(torch.int16))


def test_default_routing_on_wide_linears_agrees_with_the_oracle(ext, oracle):
    """The shapes on which the default rule leaves the first dot-product kernel (gate/up projections of
    the 7B/8B models at 3 and 6..8 bits, long rows at batch 2 and 4), against the oracle on a row slice."""
    for N, K, Ms in ((11008, 4096, (1,)), (8192, 8192, (2, 4))):
        L = make(N, K, seed=N)
        q, luts = layer_to_gpu(L)
        for b in (3, 4, 6, 8):
            for M in Ms:
                print(f"default route N={N} K={K} b={b} M={M}", flush=True)
                x, xg = _x(M, K, seed=M)
                got = ext.matmul_kbit(xg, q, luts[b], b)
                rows = slice(N - 300, N)
                _, want = oracle.matmul_kbit(x, np.ascontiguousarray(L.qweight[:, rows]), L.luts[b][rows], b, return_f64=True)
                assert_close_gemv(got[:, rows], want, f"N={N} K={K} b={b} M={M}")



def test_rows_longer_than_a_workgroup_covers(ext):
    """K beyond what one workgroup of the dot-product kernel spans (65536 at M <= 2, 32768 at 3..4):
    the entry point falls back to the MFMA kernel.  Reference: fp32 matmul of the dequantised weight."""
    gen = torch.Generator(device="cuda")
    gen.manual_seed(7)
    for K, Ms in ((66560, (1, 2)), (40960, (3, 4, 8))):
        N = 24
        q = torch.randint(-2**31, 2**31 - 1, (8, N, K // 32), dtype=torch.int32, device="cuda", generator=gen)
        for b in (3, 8):
            lut = torch.sort(torch.randn((N, 1 << b), device="cuda", generator=gen) * 0.02, dim=1).values.half()
            w = ext.dequant_kbit(q, lut, b).double()
            for M in Ms:
                print(f"long rows K={K} b={b} M={M}", flush=True)
                x = torch.randn((M, K), device="cuda", generator=gen).half()
                want = x.double() @ w.T
                got = ext.matmul_kbit(x, q, lut, b).double()
                assert (got - want).norm() <= 1e-2 * want.norm()
                assert (got - want).abs().max() <= 1e-2 * want.abs().max()


def test_denormal_table_entries_are_not_flushed(ext, oracle):
    """Tables whose entries are fp16 denormals (|w| ~ 1e-5 < 6.1e-5): every kernel must multiply them
    as they are (fp16 products, fp32 accumulate); flushing them to zero would return zeros."""
    L = make(64, 4096, seed=3)
    q, _ = layer_to_gpu(L)
    for b in (3, 5, 8):
        lut = (L.luts[b].astype(np.float32) * 5e-4).astype(np.float16)
        assert 0 < np.abs(lut).max() < 6.1e-5
        lg = torch.from_numpy(lut).cuda()
        for M, fn in ((1, ext.matmul_kbit), (2, ext.matmul_kbit), (4, ext.matmul_kbit), (8, ext.matmul_kbit),
                      (24, ext.gemm_kbit)):
            print(f"denormal tables b={b} M={M}", flush=True)
            x, xg = _x(M, L.K, seed=M)
            got = fn(xg, q, lg, b)
            _, want = oracle.matmul_kbit(x, L.qweight, lut, b, return_f64=True)
            assert np.abs(want).max() > 5e-6
            assert_close_gemv(got, want, f"denormal tables b={b} M={M}")


def test_non_finite_values_stay_where_they_belong(ext):
    """An infinite table entry makes exactly the outputs of its row infinite, an infinite activation
    exactly the outputs of its activation row -- also on rows whose last step reaches past the row end
    (K = 11008: 344 words, not a multiple of what a step of the matrix-core kernels covers), where words
    past the end must contribute zeros and not 0 * inf.  Reference: fp32 matmul of the dequantised weight."""
    N, K = 48, 11008
    L = make(N, K, seed=9)
    q, luts = layer_to_gpu(L)
    for b in (3, 8):
        lut = luts[b].clone()
        lut[5, :] = float("inf")                           # every entry of row 5
        w = ext.dequant_kbit(q, lut, b)
        for M in (1, 2, 4, 8):
            x = torch.from_numpy(synth.make_x(M, K, seed=M)).cuda().abs() + 0.01      # positive: inf rows give +inf, not NaN
            for fn in (ext.matmul_kbit, ext.gemm_kbit):
                print(f"non-finite b={b} M={M} {fn.__name__}", flush=True)
                y = fn(x, q, lut, b)
                assert torch.isinf(y[:, 5]).all() and (y[:, 5] > 0).all()
                rest = torch.cat([y[:, :5], y[:, 6:]], dim=1)
                assert torch.isfinite(rest).all()
                want = (x.double() @ w.double().T)
                want = torch.cat([want[:, :5], want[:, 6:]], dim=1)
                assert (rest.double() - want).norm() <= 1e-2 * want.norm()
            if M >= 2:
                x2 = x.clone()
                x2[1, -1] = float("inf")                   # last element of activation row 1
                y = ext.matmul_kbit(x2, q, luts[b], b)
                assert torch.isfinite(y[0]).all() and not torch.isfinite(y[1]).any()


def test_gate_and_up_with_their_activation_in_one_launch(oracle):
    """matmul_kbit_swiglu = silu(x W_gate^T) * (x W_up^T) from the oracle's float64 products; 1..4 rows, one and
    several waves per row, ragged row counts, a tail chunk (K = 11008), every bit-width.  The single rounding makes
    it closer to the float64 statement than the three-kernel path, so the usual 1e-2 bar holds with room."""
    import any_precision_ext as ext
    for N, K in ((33, 64), (100, 2048), (64, 4096), (40, 11008), (7, 8192)):
        Lg, Lu = make(N, K, seed=N + K), make(N, K, seed=N + K + 1)
        qg, lg = layer_to_gpu(Lg)
        qu, lu = layer_to_gpu(Lu)
        for b in range(3, 9):
            for M in (1, 2, 3, 4):
                print(f"swiglu N={N} K={K} b={b} M={M}", flush=True)
                x = synth.make_x(M, K, seed=M)
                xg = torch.from_numpy(x).cuda()
                got = ext.matmul_kbit_swiglu(xg, qg, lg[b], qu, lu[b], b)
                assert got.shape == (M, N) and got.dtype == torch.float16
                _, g64 = oracle.matmul_kbit(x, Lg.qweight, Lg.luts[b], b, return_f64=True)
                _, u64 = oracle.matmul_kbit(x, Lu.qweight, Lu.luts[b], b, return_f64=True)
                want = g64 / (1.0 + np.exp(-g64)) * u64
                assert_close_gemv(got, want, f"swiglu N={N} K={K} b={b} M={M}")
    with pytest.raises(ValueError, match="1..4"):
        ext.matmul_kbit_swiglu(torch.zeros((5, 8192), dtype=torch.float16, device="cuda"), qg, lg[3], qu, lu[3], 3)


def test_four_rows_per_workgroup_agree_with_the_oracle(ext, oracle):
    """At one activation row, long or many rows at low bit-widths run the dot-product kernel with four rows per
    workgroup; the knob gemv_rows = 4 forces it on small shapes (row counts that are no multiple of 4, one to
    seven waves per row, a tail chunk), and the geometry report shows where the default rule picks it."""
    from any_precision_amd import _capi
    for N, K in ((1, 64), (7, 2048), (33, 4096), (100, 11008), (18, 14336), (130, 1056)):
        L = make(N, K, seed=N + K)
        q, luts = layer_to_gpu(L)
        for b in range(3, 9):
            for M in (1, 2, 3, 4):
                print(f"four rows N={N} K={K} b={b} M={M}", flush=True)
                x, xg = _x(M, K, seed=b + M)
                with _capi.tuning(gemv_rows=4, gemv_stream=0, gemv_fine=0, matmul_mfma4=0):
                    assert _capi.matmul_geometry(M, N, K, b)["rows"] == 4 and _capi.matmul_route(M, N, K, b) == "dot"
                    got = ext.matmul_kbit(xg, q, luts[b], b)
                _, want = oracle.matmul_kbit(x, L.qweight, L.luts[b], b, return_f64=True)
                assert_close_gemv(got, want, f"N={N} K={K} b={b} M={M}")
    assert _capi.matmul_geometry(1, 14336, 4096, 3)["rows"] == 4      # 28672 waves at 3 bits
    assert _capi.matmul_geometry(1, 14336, 4096, 6)["rows"] == 2
    assert _capi.matmul_geometry(1, 14336, 4096, 8)["rows"] == 1      # one row at 8 bits on short rows
    assert _capi.matmul_geometry(1, 8192, 8192, 8)["rows"] == 4       # long rows: at every bit-width
    assert _capi.matmul_geometry(1, 4096, 11008, 3)["rows"] == 2
    assert _capi.matmul_geometry(1, 4096, 4096, 3)["rows"] == 1
    assert _capi.matmul_geometry(2, 14336, 4096, 3)["rows"] == 2      # short rows: four only at one activation row
    # 2..4 activation rows on long rows: four rows per workgroup, except rows of 5..6 waves at M = 3, 4 and of 9+ at M = 2
    # (7+ from 5 bits on); the row-streaming kernel keeps M = 3 at up to 4 bits on rows of 8 waves or more
    assert _capi.matmul_geometry(2, 4096, 14336, 5)["rows"] == 2
    for M, N, K, rows, route in ((2, 4096, 11008, 4, "dot"), (2, 4096, 14336, 4, "dot"), (3, 4096, 14336, 4, "dot"),
                                 (3, 4096, 16384, 4, "stream"),
                                 (3, 8192, 8192, 4, "dot"), (3, 4096, 11008, 2, "mfma4"), (4, 5120, 13824, 4, "dot"),
                                 (4, 28672, 8192, 4, "dot")):
        assert _capi.matmul_geometry(M, N, K, 4)["rows"] == rows and _capi.matmul_route(M, N, K, 4) == route, (M, N, K)
    assert _capi.matmul_route(4, 4096, 14336, 3) == "mfma4" and _capi.matmul_route(3, 5120, 13824, 6) == "dot"

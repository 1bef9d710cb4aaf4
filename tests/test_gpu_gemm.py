"""gemm_kbit (fused dequant -> MFMA GEMM, up to 128 rows per launch) on the GPU against the oracle,
through the C ABI.  Tolerance: 1e-2 relative (normwise and against max |y|)."""
import numpy as np
import pytest
import torch

from _util import assert_bit_exact, assert_close_gemv, layer_to_gpu, make
from any_precision_amd import synth

pytestmark = pytest.mark.gpu

RAGGED = [(1, 32), (7, 32), (5, 96), (13, 1056), (20, 2080), (130, 992), (33, 1024), (17, 3104), (21, 4128)]
SLICES = [(256, 4096), (176, 11008), (144, 14336)]
BATCHES = (1, 9, 16, 17, 40, 64, 100, 128)


@pytest.fixture(scope="module")
def ext():
    import any_precision_ext
    return any_precision_ext


def _x(M, K, seed=0):
    x = synth.make_x(M, K, seed)
    return x, torch.from_numpy(x).cuda()


@pytest.mark.parametrize("N,K", RAGGED)
def test_ragged_shapes_all_bits(ext, oracle, N, K):
    L = make(N, K, seed=N + K)
    q, luts = layer_to_gpu(L)
    for b in range(3, 9):
        for M in (1, 9, 16, 20, 32, 33, 128):
            print(f"gemm N={N} K={K} b={b} M={M}", flush=True)
            x, xg = _x(M, K, seed=M)
            got = ext.gemm_kbit(xg, q, luts[b], b)
            assert got.shape == (M, N) and got.dtype == torch.float16
            _, want = oracle.matmul_kbit(x, L.qweight, L.luts[b], b, return_f64=True)
            assert_close_gemv(got, want, f"N={N} K={K} b={b} M={M}")


@pytest.mark.parametrize("N,K", SLICES)
def test_row_slices_of_benchmark_shapes_all_batches(ext, oracle, N, K):
    L = make(N, K, seed=5)
    q, luts = layer_to_gpu(L)
    for b in range(3, 9):
        for M in BATCHES:
            print(f"gemm N={N} K={K} b={b} M={M}", flush=True)
            x, xg = _x(M, K, seed=M)
            got = ext.gemm_kbit(xg, q, luts[b], b)
            _, want = oracle.matmul_kbit(x, L.qweight, L.luts[b], b, return_f64=True)
            assert_close_gemv(got, want, f"N={N} K={K} b={b} M={M}")


@pytest.mark.parametrize("N,K", [(4096, 4096), (11008, 4096), (4096, 11008)])
def test_benchmark_shapes(ext, oracle, N, K):
    L = make(N, K, seed=1)
    q, luts = layer_to_gpu(L)
    for b in (3, 5, 8):
        for M in (16, 64):
            print(f"gemm N={N} K={K} b={b} M={M}", flush=True)
            x, xg = _x(M, K, seed=M)
            got = ext.gemm_kbit(xg, q, luts[b], b)
            _, want = oracle.matmul_kbit(x, L.qweight, L.luts[b], b, return_f64=True)
            assert_close_gemv(got, want, f"N={N} K={K} b={b} M={M}")


def test_one_hot_rows_return_dequant_columns_exactly(ext, oracle):
    # row m of x is e_{k_m}: out[m, :] is column k_m of the dequantised weight, exactly
    N, K = 48, 3104
    L = make(N, K, seed=8)
    q, luts = layer_to_gpu(L)
    ks = [0, 7, 8, 255, 256, 1023, 1024, 2047, 2048, 3071, 3072, 3080, 3103, 31, 32, 1500, 2999, 100]
    x = torch.zeros((len(ks), K), dtype=torch.float16, device="cuda")
    for m, k in enumerate(ks):
        x[m, k] = 1.0
    for b in (3, 4, 6, 8):
        w = oracle.dequant_kbit(L.qweight, L.luts[b], b)
        got = ext.gemm_kbit(x, q, luts[b], b)
        for m, k in enumerate(ks):
            assert_bit_exact(got[m], w[:, k], f"b={b} k={k}")


def test_matches_gemv_and_is_deterministic(ext):
    N, K = 512, 4096
    L = make(N, K, seed=3)
    q, luts = layer_to_gpu(L)
    _, xg = _x(8, K)
    a = ext.gemm_kbit(xg, q, luts[6], 6)
    for _ in range(3):
        assert torch.equal(ext.gemm_kbit(xg, q, luts[6], 6).view(torch.int16), a.view(torch.int16))
    v = ext.matmul_kbit(xg, q, luts[6], 6).float()
    assert (a.float() - v).norm() <= 2e-3 * v.norm()
    y3 = ext.gemm_kbit(xg.reshape(2, 4, K), q, luts[6], 6)
    assert y3.shape == (2, 4, N) and torch.equal(y3.reshape(8, N).view(torch.int16), a.view(torch.int16))


def test_more_than_128_rows_go_in_chunks_and_errors(ext, oracle):
    L = make(40, 1056, seed=0)
    q, luts = layer_to_gpu(L)
    for b, M in ((3, 129), (8, 300), (5, 512)):
        print(f"gemm chunks b={b} M={M}", flush=True)
        x, xg = _x(M, 1056, seed=M)
        got = ext.gemm_kbit(xg, q, luts[b], b)
        _, want = oracle.matmul_kbit(x, L.qweight, L.luts[b], b, return_f64=True)
        assert_close_gemv(got, want, f"b={b} M={M}")
    with pytest.raises(ValueError, match="empty"):
        ext.gemm_kbit(torch.zeros((0, 1056), dtype=torch.float16, device="cuda"), q, luts[3], 3)
    with pytest.raises(ValueError, match="float16"):
        ext.gemm_kbit(torch.zeros((16, 64), dtype=torch.float32, device="cuda"), q, luts[3], 3)


def test_graph_replay_matches_eager(ext):
    from any_precision_amd import _capi
    N, K, M = 1024, 4096, 32
    L = make(N, K, seed=4)
    q, luts = layer_to_gpu(L)
    _, xg = _x(M, K)
    eager = ext.gemm_kbit(xg, q, luts[4], 4)
    out = torch.zeros((M, N), dtype=torch.float16, device="cuda")
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        rc = _capi.lib.ap_gemm_kbit(xg.data_ptr(), q.data_ptr(), luts[4].data_ptr(), out.data_ptr(), M, N, K, 4,
                                    torch.cuda.current_stream().cuda_stream)
        assert rc == 0
    for rep in range(3):
        out.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), eager.view(torch.int16)), rep


def test_two_weight_row_blocks_per_workgroup_give_the_same_bits(ext, oracle):
    """Large linears run the MFMA kernel with two blocks of 16 weight rows per workgroup; the tuning knob
    gemm_rb2 = 2 forces that variant on the small ragged shapes a test can check against the oracle.  Each
    output is still summed in the same order, so the results must equal the one-block variant's bit for
    bit.  More than 32 activation rows go through it in chunks of 32."""
    from any_precision_amd import _capi
    shapes = ((33, 1024), (47, 2176), (130, 4096), (32, 128))
    for N, K in shapes:
        L = make(N, K, seed=N + K)
        q, luts = layer_to_gpu(L)
        for b in range(3, 9):
            for M in (9, 16, 20, 32, 40, 100):
                print(f"two row blocks N={N} K={K} b={b} M={M}", flush=True)
                x, xg = _x(M, K, seed=M)
                with _capi.tuning(gemm_rb2=2):
                    forced = ext.gemm_kbit(xg, q, luts[b], b)
                _, want = oracle.matmul_kbit(x, L.qweight, L.luts[b], b, return_f64=True)
                assert_close_gemv(forced, want, f"N={N} K={K} b={b} M={M}")
                with _capi.tuning(gemm_rb2=0):
                    plain = ext.gemm_kbit(xg, q, luts[b], b)
                assert torch.equal(plain.view(torch.int16), forced.view(torch.int16)), (N, K, b, M)


def test_lookups_one_word_ahead_give_the_same_bits(ext, oracle):
    """Linears of up to 16 rows per CU run the K-split kernel with its table lookups one word ahead of the matrix
    instructions; the knob gemm_lookahead switches the variant off (0) or forces it wherever it exists (2).  The
    order of the additions does not change, so both must give the same bits; rows of 344 and 448 words end in a
    partial step."""
    from any_precision_amd import _capi
    for N, K in ((33, 1024), (47, 2176), (176, 11008), (144, 14336), (32, 128)):
        L = make(N, K, seed=N + K)
        q, luts = layer_to_gpu(L)
        for b in range(3, 9):
            for M in (5, 9, 16, 20, 32):
                print(f"lookahead N={N} K={K} b={b} M={M}", flush=True)
                x, xg = _x(M, K, seed=M)
                with _capi.tuning(gemm_lookahead=2, gemm_rb2=0, gemm_tiled=0, gemm_walk=0):
                    ahead = ext.gemm_kbit(xg, q, luts[b], b)
                _, want = oracle.matmul_kbit(x, L.qweight, L.luts[b], b, return_f64=True)
                assert_close_gemv(ahead, want, f"N={N} K={K} b={b} M={M}")
                with _capi.tuning(gemm_lookahead=0, gemm_rb2=0, gemm_tiled=0, gemm_walk=0):
                    plain = ext.gemm_kbit(xg, q, luts[b], b)
                assert torch.equal(plain.view(torch.int16), ahead.view(torch.int16)), (N, K, b, M)


def test_row_walking_kernel_agrees_with_the_oracle(ext, oracle):
    """Wide linears at up to 32 activation rows run a variant whose workgroups walk the blocks of weight rows
    with their activations held in registers; the knob gemm_walk = 2 forces it wherever it fits (rows of a
    multiple of 128 elements, 4 to 16 steps of 512), on shapes small enough for the oracle: ragged row counts,
    a partial last step (K = 2176, 6272), one and two steps per wave (K = 8192: up to 5 bits), more blocks
    than workgroups (gemm_walk_wgs = 1 with 4112 rows on 256 CUs).  Also that it really is another kernel:
    with the knob at 0 the same call gives the one-shot kernel's result, within rounding of it."""
    from any_precision_amd import _capi
    shapes = ((48, 2048), (100, 4096), (77, 2176), (40, 6272), (33, 8192), (4112, 2048))
    for N, K in shapes:
        L = make(N, K, seed=N + K)
        q, luts = layer_to_gpu(L)
        for b in range(3, 9):
            for M in (1, 8, 16, 17, 32):
                if K > 4096 and (b > 5 or M > 16):
                    continue                     # two steps per wave exist up to 5 bits and 16 rows
                print(f"row walk N={N} K={K} b={b} M={M}", flush=True)
                x, xg = _x(M, K, seed=M)
                with _capi.tuning(gemm_walk=2):
                    walked = ext.gemm_kbit(xg, q, luts[b], b)
                _, want = oracle.matmul_kbit(x, L.qweight, L.luts[b], b, return_f64=True)
                assert_close_gemv(walked, want, f"N={N} K={K} b={b} M={M}")
                with _capi.tuning(gemm_walk=0):
                    plain = ext.gemm_kbit(xg, q, luts[b], b)
                assert_close_gemv(plain, want, f"one-shot N={N} K={K} b={b} M={M}")


def test_row_walking_kernel_on_a_wide_linear_by_default(ext, oracle):
    """14336 x 4096 at 8 bits and at 17..32 rows takes the walking kernel by the default rule; a slice of its
    outputs against the oracle on the same rows."""
    N, K = 14336, 4096
    L = make(N, K, seed=9)
    q, luts = layer_to_gpu(L)
    rows = np.r_[0:40, 7000:7040, N - 40:N]
    for b, M in ((8, 5), (8, 16), (3, 32), (5, 20)):
        print(f"row walk default N={N} K={K} b={b} M={M}", flush=True)
        x, xg = _x(M, K, seed=M)
        got = ext.gemm_kbit(xg, q, luts[b], b)
        _, want = oracle.matmul_kbit(x, L.qweight[:, rows], L.luts[b][rows], b, return_f64=True)
        assert_close_gemv(got[:, torch.from_numpy(rows).cuda()], want, f"N={N} K={K} b={b} M={M}")


def test_tiled_kernel_agrees_with_the_oracle(ext, oracle):
    """The tiled kernel (a workgroup owns 64 weight rows x 16, 32, 64 or 128 activation rows for the whole of K,
    activations staged once per workgroup in LDS) forced with gemm_tiled = 2 and every tile, on shapes small enough for
    the oracle:
    ragged row counts on both sides, one stage per byte group (K = 128), a tail chunk with a partial last step
    (K = 2176, 11008), several tiles of activation rows (M = 300).  Every output sums its products in the same order
    whatever the tile, so the two tiles agree bit for bit (with one group of waves per workgroup; with two, each on half
    of K, the sums meet in a different order)."""
    from any_precision_amd import _capi
    for N, K in ((200, 128), (64, 1024), (130, 2176), (96, 11008), (257, 4096)):
        L = make(N, K, seed=N + K)
        q, luts = layer_to_gpu(L)
        for b in range(3, 9):
            for M in (1, 17, 64, 65, 130, 300):
                print(f"tiled N={N} K={K} b={b} M={M}", flush=True)
                x, xg = _x(M, K, seed=M)
                with _capi.tuning(gemm_tiled=2, gemm_tile=4, gemm_tile_split=1):
                    small = ext.gemm_kbit(xg, q, luts[b], b)
                with _capi.tuning(gemm_tiled=2, gemm_tile=8):
                    large = ext.gemm_kbit(xg, q, luts[b], b)
                _, want = oracle.matmul_kbit(x, L.qweight, L.luts[b], b, return_f64=True)
                assert_close_gemv(small, want, f"tiled N={N} K={K} b={b} M={M}")
                assert torch.equal(small.view(torch.int16), large.view(torch.int16)), (N, K, b, M)
                # two groups of waves per workgroup, each on half of K (the second idles through a last step when
                # the number of steps is odd: K = 2176 has 5, K = 11008 has 22, K = 128 has 1 and keeps one group)
                with _capi.tuning(gemm_tiled=2, gemm_tile=4, gemm_tile_split=2):
                    halves = ext.gemm_kbit(xg, q, luts[b], b)
                assert_close_gemv(halves, want, f"tiled halves N={N} K={K} b={b} M={M}")
                # tiles of 16 and 32 activation rows (small grids; two halves of K always, so K >= 1024): the same sums
                # in the same order as the two-half form of the 64-row tile
                for tile in ((1, 2) if K >= 1024 else ()):
                    with _capi.tuning(gemm_tiled=2, gemm_tile=tile):
                        narrow = ext.gemm_kbit(xg, q, luts[b], b)
                    assert torch.equal(narrow.view(torch.int16), halves.view(torch.int16)), (N, K, b, M, tile)
    # one-hot activation rows return columns of the dequantised weight exactly (K = 2176: also the partial step)
    N, K = 130, 2176
    L = make(N, K, seed=N + K)
    q, luts = layer_to_gpu(L)
    ks = [0, 7, 8, 255, 256, 1023, 1024, 2047, 2048, 2079, 2080, 2111, 2112, 2143, 2144, 2175, 31, 32, 1500, 100] * 4
    x = torch.zeros((len(ks), K), dtype=torch.float16, device="cuda")
    for m, k in enumerate(ks):
        x[m, k] = 1.0
    for b in (3, 5, 8):
        w = oracle.dequant_kbit(L.qweight, L.luts[b], b)
        with _capi.tuning(gemm_tiled=2):
            got = ext.gemm_kbit(x, q, luts[b], b)
        for m, k in enumerate(ks):
            assert_bit_exact(got[m], w[:, k], f"tiled one-hot b={b} k={k}")


def test_tiled_kernel_by_default_beyond_128_rows(ext, oracle):
    """More than 128 activation rows on rows of a multiple of 128 elements take the tiled kernel by the default rule
    (other row lengths go in chunks of 128 through the K-split kernel): against the oracle, equal to the forced tiled
    launch bit for bit, and the same from a replayed HIP graph."""
    from any_precision_amd import _capi
    N, K = 176, 4096
    L = make(N, K, seed=11)
    q, luts = layer_to_gpu(L)
    for b, M in ((3, 129), (4, 200), (8, 300)):
        print(f"tiled default b={b} M={M}", flush=True)
        x, xg = _x(M, K, seed=M)
        got = ext.gemm_kbit(xg, q, luts[b], b)
        _, want = oracle.matmul_kbit(x, L.qweight, L.luts[b], b, return_f64=True)
        assert_close_gemv(got, want, f"tiled default b={b} M={M}")
        with _capi.tuning(gemm_tiled=2):
            forced = ext.gemm_kbit(xg, q, luts[b], b)
        assert torch.equal(got.view(torch.int16), forced.view(torch.int16))
        with _capi.tuning(gemm_tiled=0):
            chunks = ext.gemm_kbit(xg, q, luts[b], b)
        assert_close_gemv(chunks, want, f"chunks b={b} M={M}")
        out = torch.zeros((M, N), dtype=torch.float16, device="cuda")
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            rc = _capi.lib.ap_gemm_kbit(xg.data_ptr(), q.data_ptr(), luts[b].data_ptr(), out.data_ptr(), M, N, K, b,
                                        torch.cuda.current_stream().cuda_stream)
            assert rc == 0
        for rep in range(3):
            out.zero_()
            torch.cuda.synchronize()
            g.replay()
            torch.cuda.synchronize()
            assert torch.equal(out.view(torch.int16), got.view(torch.int16)), rep


def test_group_of_linears_in_one_tiled_launch(ext, oracle):
    """gemm_kbit_group: linears that share their activations (ragged row counts, a tail chunk with a partial step) in
    ONE launch of the tiled kernel -- equal to the members' own tiled launches bit for bit, as separate results and
    written side by side into one array; by the default rule (one launch beyond 32 rows, member by member below) against
    the oracle; rows of no multiple of 128 elements go member by member, and cannot be written side by side by the op
    itself (the wrapper joins them)."""
    from any_precision_amd import _capi
    for Ns, K in (((200, 64, 72), 1024), ((130, 130), 2176), ((64, 100, 40, 257), 4096)):
        Ls = [make(N, K, seed=N + K + i) for i, N in enumerate(Ns)]
        gpu = [layer_to_gpu(L) for L in Ls]
        for b in (3, 4, 6, 8):
            qs, ts = [q for q, _ in gpu], [luts[b] for _, luts in gpu]
            for M in (17, 65, 200):
                print(f"gemm group Ns={Ns} K={K} b={b} M={M}", flush=True)
                x, xg = _x(M, K, seed=M)
                with _capi.tuning(gemm_tiled=2, gemm_tile_split=1):
                    singles = [ext.gemm_kbit(xg, q, t, b) for q, t in zip(qs, ts)]
                    outs = ext.gemm_kbit_group(xg, qs, ts, b)
                    joint = ext.gemm_kbit_group(xg, qs, ts, b, concat=True)
                for s_, o in zip(singles, outs):
                    assert torch.equal(s_.view(torch.int16), o.view(torch.int16))
                assert joint.shape == (M, sum(Ns)) and torch.equal(joint, torch.cat(singles, dim=-1))
                outs = ext.gemm_kbit_group(xg, qs, ts, b)                  # default rule
                for L, o in zip(Ls, outs):
                    _, want = oracle.matmul_kbit(x, L.qweight, L.luts[b], b, return_f64=True)
                    assert_close_gemv(o, want, f"group Ns={Ns} K={K} b={b} M={M} N={L.N}")
    # K = 1056: the tiled kernel does not serve it
    Ls = [make(N, 1056, seed=N) for N in (40, 24)]
    gpu = [layer_to_gpu(L) for L in Ls]
    x, xg = _x(50, 1056, seed=3)
    qs, ts = [q for q, _ in gpu], [luts[5] for _, luts in gpu]
    joint = ext.gemm_kbit_group(xg, qs, ts, 5, concat=True)
    for L, o in zip(Ls, torch.split(joint, [40, 24], dim=-1)):
        _, want = oracle.matmul_kbit(x, L.qweight, L.luts[5], 5, return_f64=True)
        assert_close_gemv(o, want, f"group K=1056 N={L.N}")
    out = torch.empty((50, 64), dtype=torch.float16, device="cuda")
    rc = _capi.gemm_group(xg.data_ptr(), [q.data_ptr() for q in qs], [t.data_ptr() for t in ts],
                          [out.data_ptr(), out.data_ptr() + 80], [40, 24], [64, 64], 50, 1056, 5, torch.cuda.current_stream().cuda_stream)
    assert rc == _capi.AP_ESHAPE
    q8, luts8 = layer_to_gpu(make(8, 64, seed=1))
    with pytest.raises(ValueError, match="same in_features"):
        ext.gemm_kbit_group(xg, [qs[0], q8], [ts[0], luts8[5]], 5)

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


def test_grouped_launch_is_bit_identical_to_the_separate_calls(ext, oracle):
    """dequant_kbit_group: up to eight linears of different shapes in one launch (ragged rows, tail chunks, a
    member of one segment, members larger than a grid round) against the oracle and the single calls."""
    from any_precision_amd import _capi
    shapes = [(13, 1056), (1, 32), (130, 992), (4, 2080), (640, 4096), (96, 11008), (7, 32), (33, 1024)]
    layers = [make(N, K, seed=3 * N + K) for N, K in shapes]
    on_gpu = [layer_to_gpu(L) for L in layers]
    for b in range(3, 9):
        for count in (1, 2, 7, 8):
            print(f"dequant group b={b} count={count}", flush=True)
            got = ext.dequant_kbit_group([q for q, _ in on_gpu[:count]], [t[b] for _, t in on_gpu[:count]], b)
            assert len(got) == count
            for g, (L, (q, luts)) in enumerate(zip(layers[:count], on_gpu[:count])):
                assert_bit_exact(got[g], oracle.dequant_kbit(L.qweight, L.luts[b], b), f"member {g} b={b} count={count}")
                assert torch.equal(got[g].view(torch.int16), ext.dequant_kbit(q, luts[b], b).view(torch.int16))
    # a small grid (one workgroup per CU): every wave strides through several members
    with _capi.tuning(dequant_blocks_per_cu=1):
        got = ext.dequant_kbit_group([q for q, _ in on_gpu], [t[5] for _, t in on_gpu], 5)
    for g, L in enumerate(layers):
        assert_bit_exact(got[g], oracle.dequant_kbit(L.qweight, L.luts[5], 5), f"strided member {g}")
    with pytest.raises(ValueError):
        ext.dequant_kbit_group([on_gpu[0][0]] * 9, [on_gpu[0][1][3]] * 9, 3)


def test_grouped_launch_over_a_decoder_layer_set(ext):
    """The seven linears of a Llama-2-7B layer in one launch against the single calls, bit for bit (random planes)."""
    from any_precision_amd import synth
    gen = torch.Generator(device="cuda")
    gen.manual_seed(11)
    qs = [torch.randint(-2**31, 2**31 - 1, (8, N, K // 32), dtype=torch.int32, device="cuda", generator=gen)
          for _, N, K in synth.LLAMA2_7B_LAYER]
    for b in (3, 8):
        ts = [torch.sort(torch.randn((N, 1 << b), device="cuda", generator=gen) * 0.02, dim=1).values.half()
              for _, N, K in synth.LLAMA2_7B_LAYER]
        got = ext.dequant_kbit_group(qs, ts, b)
        for g, (q, t) in enumerate(zip(qs, ts)):
            assert torch.equal(got[g].view(torch.int16), ext.dequant_kbit(q, t, b).view(torch.int16)), f"member {g} b={b}"
        del got


def test_grouped_launch_replays_in_a_graph(ext):
    """One ap_dequant_kbit_group launch captured in a HIP graph (members travel as kernel arguments: nothing to copy at
    replay) against the eager result on every replay, with eager work and synchronisations between the replays."""
    shapes = [(96, 4096), (64, 11008), (33, 1024)]
    layers = [make(N, K, seed=7 * N + K) for N, K in shapes]
    on_gpu = [layer_to_gpu(L) for L in layers]
    b = 5
    qs, ts = [q for q, _ in on_gpu], [t[b] for _, t in on_gpu]
    want = ext.dequant_kbit_group(qs, ts, b)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            got = ext.dequant_kbit_group(qs, ts, b)
    for rep in range(3):
        for g in got:
            g.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for g, (a, w) in enumerate(zip(got, want)):
            assert torch.equal(a.view(torch.int16), w.view(torch.int16)), f"replay {rep} member {g}"
        _ = ext.dequant_kbit(qs[0], ts[0], b)      # eager work between the replays

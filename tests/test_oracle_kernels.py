"""Pins of the oracle's per-lane transpose and GEMV (CPU only)."""
import numpy as np
import pytest


def _index_by_definition(q, bits, pos):
    """index of the element stored at word bit `pos`: plane 0 is the MSB."""
    v = 0
    for p in range(bits):
        v = (v << 1) | ((int(q[p]) >> pos) & 1)
    return v


@pytest.mark.parametrize("bits", range(1, 9))
def test_transpose_against_definition(oracle, bits):
    rng = np.random.default_rng(bits)
    for _ in range(50):
        q = rng.integers(0, 2**32, size=bits, dtype=np.uint64).astype(np.uint32)
        q_w = oracle.transpose(q, bits)
        for e in range(8):
            for c in range(4):
                assert (int(q_w[e]) >> (8 * c)) & 0xff == _index_by_definition(q, bits, 8 * c + 7 - e)


@pytest.mark.parametrize("bits", [3, 4])
def test_pair_transpose_is_two_indices_per_byte(oracle, bits):
    rng = np.random.default_rng(10 + bits)
    for _ in range(50):
        q = rng.integers(0, 2**32, size=bits, dtype=np.uint64).astype(np.uint32)
        s = oracle.transpose(q, bits)
        pw = oracle.transpose_pair(q, bits)
        for m in range(4):
            for c in range(4):
                hi = (int(s[m]) >> (8 * c)) & 0xff
                lo = (int(s[m + 4]) >> (8 * c)) & 0xff
                assert (int(pw[m]) >> (8 * c)) & 0xff == (hi << bits) | lo


def test_transpose_single_bit_walk(oracle):
    # one set bit in one plane lands in exactly one index bit
    for bits in (3, 5, 8):
        for p in range(bits):
            for pos in range(32):
                q = np.zeros(bits, dtype=np.uint32)
                q[p] = np.uint32(1 << pos)
                q_w = oracle.transpose(q, bits)
                c, u = divmod(pos, 8)
                expect = np.zeros(8, dtype=np.uint32)
                expect[7 - u] = np.uint32(1 << (8 * c + bits - 1 - p))
                assert np.array_equal(q_w, expect)


def test_half_conversions_roundtrip_all_values(oracle):
    L = oracle.lib()
    allh = np.arange(65536, dtype=np.uint16)
    want = allh.view(np.float16).astype(np.float32)
    for h in range(0, 65536, 7):
        f = L.apo_half_to_float(h)
        if np.isnan(want[h]):
            assert np.isnan(f)
            continue
        assert np.float32(f) == want[h]
        assert L.apo_double_to_half(float(f)) == h or (h == 0x8000 and L.apo_double_to_half(float(f)) == 0x8000)


def test_double_to_half_rounds_like_numpy(oracle):
    L = oracle.lib()
    rng = np.random.default_rng(0)
    vals = np.concatenate([rng.normal(0, 1, 4000), rng.normal(0, 1e-5, 2000), rng.normal(0, 3e4, 2000),
                           np.array([65504.0, 65519.9, 65520.0, 1e9, 5.96e-8, 2.98e-8, 2.99e-8, 0.0, -0.0,
                                     6.1e-5, 6.097e-5, 0.333251953125 + 2**-13])])
    for v in vals:
        got = L.apo_double_to_half(float(v))
        with np.errstate(over="ignore"):
            want = int(np.float64(v).astype(np.float16).view(np.uint16))
        assert got == want, v


SHAPES = [(8, 32), (4, 96), (5, 1056), (16, 4096), (3, 11008)]


@pytest.mark.parametrize("N,K", SHAPES)
def test_gemv_is_matmul_of_dequantised_weights(oracle, N, K):
    rng = np.random.default_rng(N * K)
    codes = rng.integers(0, 256, size=(N, K), dtype=np.uint8)
    qw = oracle.pack_bitplanes(codes, 8)
    for b in (3, 5, 8):
        lut = np.sort(rng.normal(0, 0.02, size=(N, 1 << b)), axis=1).astype(np.float16)
        w = np.take_along_axis(lut, (codes >> (8 - b)).astype(np.int64), axis=1).astype(np.float64)
        for M in (1, 3, 8):
            x = rng.normal(0, 1, size=(M, K)).astype(np.float16)
            y16, y64 = oracle.matmul_kbit(x, qw, lut, b, return_f64=True)
            want = x.astype(np.float64) @ w.T
            assert np.allclose(y64, want, rtol=1e-12, atol=1e-13)
            with np.errstate(over="ignore"):
                assert np.array_equal(y16.view(np.uint16), want.astype(np.float16).view(np.uint16)) or \
                    np.allclose(y16.astype(np.float64), want, rtol=1e-3)   # double rounding differs by <= 1 ulp
            fast = oracle.matmul_kbit_fast(x, qw, lut, b)
            assert np.linalg.norm(fast.astype(np.float64) - want) <= 2e-3 * np.linalg.norm(want) + 1e-6


def test_gemv_one_hot_x_gives_dequant_column(oracle):
    rng = np.random.default_rng(5)
    N, K = 7, 2080
    codes = rng.integers(0, 256, size=(N, K), dtype=np.uint8)
    qw = oracle.pack_bitplanes(codes, 8)
    for b in (3, 4, 7):
        lut = rng.normal(0, 0.02, size=(N, 1 << b)).astype(np.float16)
        w = oracle.dequant_kbit(qw, lut, b)
        for k in (0, 7, 8, 255, 256, 1023, 1024, 2047, 2048, 2079):
            x = np.zeros((1, K), dtype=np.float16)
            x[0, k] = 1.0
            y = oracle.matmul_kbit(x, qw, lut, b)
            assert np.array_equal(y[0].view(np.uint16), w[:, k].view(np.uint16)), (b, k)


def test_gemv_constant_table_gives_scaled_sum_of_x(oracle):
    rng = np.random.default_rng(6)
    N, K = 4, 1056
    codes = rng.integers(0, 256, size=(N, K), dtype=np.uint8)
    qw = oracle.pack_bitplanes(codes, 8)
    x = rng.normal(0, 1, size=(2, K)).astype(np.float16)
    lut = np.full((N, 32), 0.5, dtype=np.float16)
    _, y64 = oracle.matmul_kbit(x, qw, lut, 5, return_f64=True)
    want = 0.5 * x.astype(np.float64).sum(axis=1, keepdims=True) * np.ones((1, N))
    assert np.allclose(y64, want, rtol=1e-13, atol=1e-13)


def test_gemv_linear_in_x(oracle):
    rng = np.random.default_rng(8)
    N, K = 5, 1024
    codes = rng.integers(0, 256, size=(N, K), dtype=np.uint8)
    qw = oracle.pack_bitplanes(codes, 8)
    lut = rng.normal(0, 0.02, size=(N, 64)).astype(np.float16)
    a = rng.integers(-8, 8, size=(1, K)).astype(np.float16)
    b = rng.integers(-8, 8, size=(1, K)).astype(np.float16)
    _, ya = oracle.matmul_kbit(a, qw, lut, 6, return_f64=True)
    _, yb = oracle.matmul_kbit(b, qw, lut, 6, return_f64=True)
    _, yab = oracle.matmul_kbit((a + 2 * b).astype(np.float16), qw, lut, 6, return_f64=True)
    assert np.allclose(yab, ya + 2 * yb, rtol=1e-12, atol=1e-12)


def test_leading_dims_are_batch(oracle):
    rng = np.random.default_rng(9)
    codes = rng.integers(0, 256, size=(4, 64), dtype=np.uint8)
    qw = oracle.pack_bitplanes(codes, 8)
    lut = rng.normal(0, 0.02, size=(4, 8)).astype(np.float16)
    x = rng.normal(0, 1, size=(2, 3, 64)).astype(np.float16)
    y = oracle.matmul_kbit(x, qw, lut, 3)
    assert y.shape == (2, 3, 4)
    assert np.array_equal(y.reshape(6, 4), oracle.matmul_kbit(x.reshape(6, 64), qw, lut, 3))

"""The kernels' pure-integer helpers (ap_bitplane.hpp), built for the host with
g++, against the oracle and against the layout definition (CPU only)."""
import ctypes

import numpy as np
import pytest


def _run(hostcheck, q, bits, shift=0):
    q = np.ascontiguousarray(q, dtype=np.uint32)
    out = np.zeros(8, dtype=np.uint32)
    rc = hostcheck.aph_planes_to_indices(ctypes.c_void_p(q.ctypes.data), bits, shift, ctypes.c_void_p(out.ctypes.data))
    assert rc == 0
    return out


@pytest.mark.parametrize("bits", range(1, 9))
def test_butterfly_transpose_matches_oracle(hostcheck, oracle, bits):
    rng = np.random.default_rng(bits)
    for _ in range(300):
        q = rng.integers(0, 2**32, size=bits, dtype=np.uint64).astype(np.uint32)
        assert np.array_equal(_run(hostcheck, q, bits), oracle.transpose(q, bits))
    for p in range(bits):                    # walking ones / zeros
        for pos in range(32):
            q = np.zeros(bits, dtype=np.uint32)
            q[p] = np.uint32(1 << pos)
            assert np.array_equal(_run(hostcheck, q, bits), oracle.transpose(q, bits))
            q = ~q
            assert np.array_equal(_run(hostcheck, q, bits), oracle.transpose(q, bits))


@pytest.mark.parametrize("bits", range(3, 8))
def test_preshifted_indices(hostcheck, oracle, bits):
    rng = np.random.default_rng(40 + bits)
    for _ in range(100):
        q = rng.integers(0, 2**32, size=bits, dtype=np.uint64).astype(np.uint32)
        assert np.array_equal(_run(hostcheck, q, bits, 1), oracle.transpose(q, bits) << np.uint32(1))


@pytest.mark.parametrize("bits", [3, 4])
def test_adjacent_pair_indices(hostcheck, oracle, bits):
    """Byte b of apair[i] names the table entry of elements (2i, 2i+1) of byte group 3 - b: splitting it
    must give back the two indices the oracle's transpose holds for those elements (idx[e] byte b)."""
    rng = np.random.default_rng(70 + bits)
    first, second = ctypes.c_uint32(), ctypes.c_uint32()
    for trial in range(200):
        q = rng.integers(0, 2**32, size=bits, dtype=np.uint64).astype(np.uint32)
        if trial < bits * 2:                 # walking planes: all ones / a single one
            q = np.zeros(bits, dtype=np.uint32)
            q[trial % bits] = np.uint32(0xFFFFFFFF if trial < bits else 1 << (5 * trial % 32))
        out = np.zeros(4, dtype=np.uint32)
        assert hostcheck.aph_planes_to_adjacent_pairs(ctypes.c_void_p(q.ctypes.data), bits,
                                                      ctypes.c_void_p(out.ctypes.data)) == 0
        want = oracle.transpose(q, bits)     # want[e] byte b = index of element e of that byte
        for i in range(4):
            for b in range(4):
                byte = (int(out[i]) >> (8 * b)) & 0xFF
                if bits == 3:
                    assert byte % 4 == 0     # a dword offset into 64 entries
                assert hostcheck.aph_adjacent_pair_split(bits, byte, ctypes.byref(first), ctypes.byref(second)) == 0
                assert first.value == (int(want[2 * i]) >> (8 * b)) & 0xFF, (i, b)
                assert second.value == (int(want[2 * i + 1]) >> (8 * b)) & 0xFF, (i, b)


@pytest.mark.parametrize("K", [32, 64, 992, 1024, 1056, 4096, 11008, 14336])
def test_group_base_enumerates_every_element_once(hostcheck, K):
    W = K // 32
    seen = np.zeros(K, dtype=np.int32)
    for w in range(W):
        T = hostcheck.aph_chunk_words(w, K)
        assert T == (32 if (w // 32) < K // 1024 else (K % 1024) // 32)
        for j in range(4):
            k0 = hostcheck.aph_group_base(w, j, K)
            assert k0 % 8 == 0 and 0 <= k0 <= K - 8
            seen[k0:k0 + 8] += 1
    assert (seen == 1).all()


def test_group_base_matches_packer(hostcheck, oracle):
    # a one-hot code at element k must show up in word w, byte group j, bit e as the helper says
    K = 1056 + 64
    W = K // 32
    where = {}
    for w in range(W):
        for j in range(4):
            k0 = hostcheck.aph_group_base(w, j, K)
            for e in range(8):
                where[k0 + e] = (w, 8 * (3 - j) + 7 - e)
    rng = np.random.default_rng(1)
    for k in rng.choice(K, size=80, replace=False):
        codes = np.zeros((1, K), dtype=np.uint8)
        codes[0, k] = 0x80
        qw = oracle.pack_bitplanes(codes, 8).view(np.uint32)[0, 0]
        w, bit = where[int(k)]
        expect = np.zeros(W, dtype=np.uint32)
        expect[w] = np.uint32(1 << bit)
        assert np.array_equal(qw, expect)


def test_division_by_host_reciprocal_is_exact(hostcheck):
    """The kernels divide by a run-time divisor with a reciprocal from the launch code (ap_reciprocal.hpp).
    Against Python's integer division: every divisor up to 600 with numerators around every multiple boundary and
    at the top of the range, and random pairs over the whole range the kernels allow."""
    q, r = ctypes.c_uint32(), ctypes.c_uint32()
    rng = np.random.default_rng(7)
    top = 2**31 - 1
    for d in list(range(1, 601)) + [1023, 1024, 4097, 65535, 65536, 2**20 + 1, 2**30, top]:
        ns = {0, 1, d - 1, d, d + 1, top, top - 1, (top // d) * d, max((top // d) * d - 1, 0)}
        ns |= {int(k) * d + o for k in rng.integers(0, max(top // d, 1), size=6) for o in (-1, 0, 1)}
        for n in ns:
            if 0 <= n <= top:
                assert hostcheck.aph_divmod_by_reciprocal(n, d, ctypes.byref(q), ctypes.byref(r)) == 0
                assert (q.value, r.value) == divmod(n, d), (n, d)
    for n, d in zip(rng.integers(0, 2**31, size=20000), rng.integers(1, 2**31, size=20000)):
        assert hostcheck.aph_divmod_by_reciprocal(int(n), int(d), ctypes.byref(q), ctypes.byref(r)) == 0
        assert (q.value, r.value) == divmod(int(n), int(d)), (n, d)
    # the K-split form: no correction step, exact while n * d < 2^32
    for d in range(1, 17):
        lim = 2**32 // d
        ns = {0, 1, d - 1, d, lim - 1, lim - 2, (lim - 1) // d * d, (lim - 1) // d * d - 1}
        ns |= {int(v) for v in rng.integers(0, lim, size=4000)}
        for n in ns:
            if 0 <= n < lim:
                assert hostcheck.aph_div_by_reciprocal_ceil(n, d, ctypes.byref(q)) == 0
                assert q.value == n // d, (n, d)
    assert hostcheck.aph_div_by_reciprocal_ceil(2**31, 2, ctypes.byref(q)) == -1   # outside the exact range: refused
    assert hostcheck.aph_divmod_by_reciprocal(2**31, 3, ctypes.byref(q), ctypes.byref(r)) == -1

"""Pins of the oracle's layout functions (CPU only).

What is checked against what:
* hand-derived known answers for K=32 and K=64 (worked out from pack.py on paper);
* the C packer against the numpy statement of pack.py (packbits + argsort);
* pack (follows pack.py) -> dequant (follows the kernel's addressing in
  dequant.cuh) == lut[code >> (P - b)] (eval.py:104-105): two independent
  reference sources must agree;
* prefix property index_b == index_{b+1} >> 1;
* every code value at every one of the 32 positions of a word.
"""
import numpy as np
import pytest

KS = [32, 64, 96, 992, 1024, 1056, 2048, 4096, 11008, 14336]


def _u32(a):
    return np.ascontiguousarray(a).view(np.uint32)


def test_kat_k32_counting_codes(oracle):
    # K=32: one word, tail chunk with T=1 -> element k sits at bit 31-k.
    # codes[k] = k: plane of bit v is the MSB-first bit string of (k >> v) & 1.
    codes = np.arange(32, dtype=np.uint8)[None, :]
    qw = _u32(oracle.pack_bitplanes(codes, 8))
    assert qw.shape == (8, 1, 1)
    expect = {7: 0x55555555, 6: 0x33333333, 5: 0x0F0F0F0F, 4: 0x00FF00FF, 3: 0x0000FFFF, 2: 0, 1: 0, 0: 0}
    for plane, word in expect.items():
        assert int(qw[plane, 0, 0]) == word, plane


def test_kat_k64_single_elements(oracle):
    # K=64: T=2.  Element k = 8*(2j+t)+e sits in word t at bit 8*(3-j)+(7-e).
    for k in range(64):
        codes = np.zeros((1, 64), dtype=np.uint8)
        codes[0, k] = 0x80                      # only plane 0 (MSB) is set
        qw = _u32(oracle.pack_bitplanes(codes, 8))
        byte, e = divmod(k, 8)
        j, t = divmod(byte, 2)
        word = [0, 0]
        word[t] = 1 << (8 * (3 - j) + 7 - e)
        assert [int(v) for v in qw[0, 0]] == word, k
        assert not qw[1:].any()


def test_kat_full_chunk_single_elements(oracle):
    # K=1024: T=32, k = 256 j + 8 t + e -> word t, bit 8(3-j)+(7-e); plane p holds code bit 7-p.
    rng = np.random.default_rng(0)
    for k in rng.choice(1024, size=64, replace=False):
        for p in (0, 3, 7):
            codes = np.zeros((2, 1024), dtype=np.uint8)
            codes[1, k] = 1 << (7 - p)
            qw = _u32(oracle.pack_bitplanes(codes, 8))
            j, rem = divmod(int(k), 256)
            t, e = divmod(rem, 8)
            expect = np.zeros((8, 2, 32), dtype=np.uint32)
            expect[p, 1, t] = 1 << (8 * (3 - j) + 7 - e)
            assert np.array_equal(qw, expect)


@pytest.mark.parametrize("K", KS)
def test_c_packer_matches_numpy_statement_of_pack_py(oracle, K):
    rng = np.random.default_rng(K)
    codes = rng.integers(0, 256, size=(5, K), dtype=np.uint8)
    assert np.array_equal(oracle.pack_bitplanes(codes, 8), oracle.np_pack_bitplanes(codes, 8))


@pytest.mark.parametrize("P", [3, 4, 6, 8])
def test_packers_agree_for_smaller_parents(oracle, P):
    rng = np.random.default_rng(P)
    codes = rng.integers(0, 1 << P, size=(3, 1056), dtype=np.uint8)
    a = oracle.pack_bitplanes(codes, P)
    assert a.shape == (P, 3, 33)
    assert np.array_equal(a, oracle.np_pack_bitplanes(codes, P))


@pytest.mark.parametrize("K", KS)
def test_pack_then_dequant_is_table_lookup_of_top_bits(oracle, K):
    rng = np.random.default_rng(100 + K)
    N = 6
    codes = rng.integers(0, 256, size=(N, K), dtype=np.uint8)
    qw = oracle.np_pack_bitplanes(codes, 8)          # pack.py statement
    for b in range(3, 9):
        lut = rng.normal(0, 0.02, size=(N, 1 << b)).astype(np.float16)
        got = oracle.dequant_kbit(qw, lut, b)        # kernel-addressing statement
        want = np.take_along_axis(lut, (codes >> (8 - b)).astype(np.int64), axis=1)
        assert np.array_equal(got.view(np.uint16), want.view(np.uint16)), b


def test_dequant_reads_only_top_planes(oracle):
    rng = np.random.default_rng(7)
    codes = rng.integers(0, 256, size=(4, 2080), dtype=np.uint8)
    qw = oracle.pack_bitplanes(codes, 8)
    for b in range(3, 8):
        lut = rng.normal(0, 1, size=(4, 1 << b)).astype(np.float16)
        full = oracle.dequant_kbit(qw, lut, b)
        pruned = oracle.dequant_kbit(qw[:b].copy(), lut, b)   # AnyPrecisionLinear.prune_precisions
        scrambled = qw.copy()
        scrambled[b:] = rng.integers(-2**31, 2**31 - 1, size=scrambled[b:].shape, dtype=np.int64).astype(np.int32)
        assert np.array_equal(full.view(np.uint16), pruned.view(np.uint16))
        assert np.array_equal(full.view(np.uint16), oracle.dequant_kbit(scrambled, lut, b).view(np.uint16))


def test_prefix_property(oracle):
    # identity tables turn dequant into the index itself
    rng = np.random.default_rng(3)
    codes = rng.integers(0, 256, size=(3, 1120), dtype=np.uint8)
    qw = oracle.pack_bitplanes(codes, 8)
    idx = {}
    for b in range(3, 9):
        ident = np.tile(np.arange(1 << b, dtype=np.float16), (3, 1))
        idx[b] = oracle.dequant_kbit(qw, ident, b).astype(np.int64)
        assert np.array_equal(idx[b], codes >> (8 - b))
    for b in range(3, 8):
        assert np.array_equal(idx[b], idx[b + 1] >> 1)


def test_every_code_at_every_word_position(oracle):
    # 256 codes x 32 positions of one word (K=32), and of a word inside a full chunk
    for K, base in ((32, 0), (1024, 8 * 5)):
        ident = np.arange(256, dtype=np.float16)[None, :]
        for pos in range(32):
            codes = np.zeros((256, K), dtype=np.uint8)
            # position pos of word 0 (K=32) / of word t=5 (K=1024): element index by layout
            if K == 32:
                k = pos
            else:
                j, e = divmod(pos, 8)
                k = 256 * j + base + e
            codes[:, k] = np.arange(256, dtype=np.uint8)
            qw = oracle.pack_bitplanes(codes, 8)
            out = oracle.dequant_kbit(qw, np.tile(ident, (256, 1)), 8)
            assert np.array_equal(out[:, k].astype(np.int64), np.arange(256))
            out[:, k] = 0
            assert not out.any()

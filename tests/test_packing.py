"""The package's numpy packer against the oracle packers (CPU only)."""
import numpy as np
import pytest

from any_precision_amd import packing, synth


@pytest.mark.parametrize("K", [32, 64, 992, 1024, 1056, 4096, 11008])
def test_pack_codes_matches_oracle(oracle, K):
    rng = np.random.default_rng(K)
    codes = rng.integers(0, 256, size=(4, K), dtype=np.uint8)
    got = packing.pack_codes(codes, 8)
    assert got.dtype == np.int32 and got.shape == (8, 4, K // 32)
    assert np.array_equal(got, oracle.pack_bitplanes(codes, 8))
    assert np.array_equal(got, oracle.np_pack_bitplanes(codes, 8))


@pytest.mark.parametrize("P", [3, 5, 8])
def test_unpack_inverts_pack_and_prefixes(P):
    rng = np.random.default_rng(P)
    codes = rng.integers(0, 1 << P, size=(3, 2080), dtype=np.uint8)
    qw = packing.pack_codes(codes, P)
    assert np.array_equal(packing.unpack_codes(qw), codes)
    for b in range(1, P + 1):
        assert np.array_equal(packing.unpack_codes(qw, b), codes >> (P - b))
        assert np.array_equal(packing.unpack_codes(qw[:b], b), codes >> (P - b))


def test_pack_rejects_bad_input():
    with pytest.raises(ValueError):
        packing.pack_codes(np.zeros((2, 40), dtype=np.uint8))
    with pytest.raises(ValueError):
        packing.pack_codes(np.full((2, 32), 9, dtype=np.uint8), parent_bits=3)
    with pytest.raises(ValueError):
        packing.unpack_codes(np.zeros((3, 2, 1), dtype=np.int32), 4)


def test_pack_layer_keys_and_shapes():
    L = synth.make_layer(8, 64, seed=0)
    entries = packing.pack_layer(L.codes, L.luts)
    assert sorted(entries) == ["lut3", "lut4", "lut5", "lut6", "lut7", "lut8", "qweight"]
    assert entries["qweight"].shape == (8, 8, 2) and entries["qweight"].dtype == np.int32
    for b in range(3, 9):
        assert entries[f"lut{b}"].shape == (8, 1 << b) and entries[f"lut{b}"].dtype == np.float16
    with pytest.raises(ValueError):
        packing.pack_layer(L.codes, {3: np.zeros((8, 4), dtype=np.float16)})


def test_synth_layer_is_seeded_and_sorted():
    a, b = synth.make_layer(16, 96, seed=3), synth.make_layer(16, 96, seed=3)
    assert np.array_equal(a.qweight, b.qweight)
    for bits in range(3, 9):
        assert np.array_equal(a.luts[bits], b.luts[bits])
        assert (np.diff(a.luts[bits].astype(np.float32), axis=1) >= 0).all()
    assert not np.array_equal(a.codes, synth.make_layer(16, 96, seed=4).codes)
    assert synth.gemv_bytes(4096, 4096, 3) == 6_373_376      # 6.373 MB, the figure the roofline uses
    assert synth.dequant_bytes(4096, 4096, 8) == 16_777_216 + 2_097_152 + 33_554_432

#!/usr/bin/env python3
"""Writes tests/golden/bitplane_small.npz: small seeded layers in the checkpoint layout with
their expected dequantised weights and GEMV results.

The reference ships no fixtures and cannot run here (its packer needs numba, its kernels
CUDA), so the vectors come from this repository's own statements of the reference:
``qweight`` from ``any_precision_amd.packing.pack_codes`` (pack.py:12-76,90-99), ``w{b}`` from
the definition ``lut[code >> (8 - b)]`` (eval.py:104-105), ``y{b}`` from a float64 matmul of
those.  tests/test_golden.py checks the C oracle, the numpy packer and the HIP library
against them; the file is regenerated only when the format itself is extended.

    python tests/golden/make_vectors.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "..", "..", "any-precision-llm_amd"))

from any_precision_amd.packing import pack_codes  # noqa: E402

SHAPES = [(3, 32), (5, 96), (4, 1056), (6, 2080), (2, 3104)]   # ragged rows, one to three chunks, tails 1..2 words
M = 3


def main():
    out = {"shapes": np.array(SHAPES, dtype=np.int64)}
    for i, (N, K) in enumerate(SHAPES):
        rng = np.random.default_rng(1000 + i)
        codes = rng.integers(0, 256, size=(N, K), dtype=np.uint8)
        x = rng.normal(0, 1, size=(M, K)).astype(np.float16)
        out[f"s{i}_codes"] = codes
        out[f"s{i}_qweight"] = pack_codes(codes, 8)
        out[f"s{i}_x"] = x
        for b in range(3, 9):
            lut = np.sort(rng.normal(0, 0.02, size=(N, 1 << b)), axis=1).astype(np.float16)
            w = np.take_along_axis(lut, (codes >> (8 - b)).astype(np.int64), axis=1)
            out[f"s{i}_lut{b}"] = lut
            out[f"s{i}_w{b}"] = w
            out[f"s{i}_y{b}"] = x.astype(np.float64) @ w.astype(np.float64).T
    path = os.path.join(HERE, "bitplane_small.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()

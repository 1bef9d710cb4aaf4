"""Bitplane checkpoint layout: pack parent codes into ``qweight`` and back.

Vectorised numpy counterpart of the reference packer
(any_precision/quantization/pack.py:12-76 permutation, :90-99 plane order):

* ``qweight`` is int32 ``[P, N, K/32]``; plane 0 is the MSB of the parent code.
* A row is cut into chunks of 1024 elements (32 words); a last partial chunk
  holds ``T = (K % 1024) / 32`` words.  Word ``t`` of chunk ``c``, read as
  uint32 from MSB to LSB, holds elements ``1024 c + 8 (T j + t) + e`` for
  ``j = 0..3`` (byte groups) and ``e = 0..7``.
"""
from __future__ import annotations

import numpy as np

CHUNK = 1024


def _chunks(K: int):
    """(first element, words in chunk) for every chunk of a row."""
    full = K // CHUNK
    out = [(c * CHUNK, 32) for c in range(full)]
    if K % CHUNK:
        out.append((full * CHUNK, (K % CHUNK) // 32))
    return out


def pack_codes(codes: np.ndarray, parent_bits: int = 8) -> np.ndarray:
    """uint8 ``[N, K]`` parent codes (< 2**parent_bits) -> int32 ``[P, N, K/32]``."""
    codes = np.ascontiguousarray(codes, dtype=np.uint8)
    if codes.ndim != 2 or codes.shape[1] % 32 != 0:
        raise ValueError(f"codes must be [N, K] with K a multiple of 32, got {codes.shape}")
    if not 1 <= parent_bits <= 8:
        raise ValueError("parent_bits must be in 1..8")
    if parent_bits < 8 and codes.size and int(codes.max()) >> parent_bits:
        raise ValueError("code value does not fit parent_bits")
    N, K = codes.shape
    out = np.empty((parent_bits, N, K // 32), dtype=np.uint32)
    for p in range(parent_bits):
        bits = (codes >> (parent_bits - 1 - p)) & 1                     # [N, K]
        for k0, T in _chunks(K):
            blk = bits[:, k0:k0 + 32 * T].reshape(N, 4, T, 8)          # [n, j, t, e]
            blk = blk.transpose(0, 2, 1, 3).reshape(N, T, 32)           # [n, t, (j e)] MSB first
            by = np.packbits(blk, axis=-1)                              # [n, t, 4] big-endian bytes
            out[p, :, k0 // 32:k0 // 32 + T] = by.view(">u4").reshape(N, T)
    return out.view(np.int32)


def unpack_codes(qweight: np.ndarray, bits: int | None = None) -> np.ndarray:
    """int32 ``[P', N, K/32]`` -> uint8 ``[N, K]`` built from planes ``0..bits-1``
    (``bits`` defaults to all planes held): the ``bits``-bit index of every element."""
    qw = np.ascontiguousarray(qweight).view(np.uint32)
    P, N, W = qw.shape
    bits = P if bits is None else bits
    if not 1 <= bits <= P:
        raise ValueError(f"bits={bits} outside 1..{P}")
    K = W * 32
    idx = np.zeros((N, K), dtype=np.uint8)
    for p in range(bits):
        for k0, T in _chunks(K):
            words = qw[p, :, k0 // 32:k0 // 32 + T]                     # [n, t]
            by = words.astype(">u4").view(np.uint8).reshape(N, T, 4)    # byte j of word t
            b = np.unpackbits(by, axis=-1).reshape(N, T, 4, 8)          # [n, t, j, e]
            b = b.transpose(0, 2, 1, 3).reshape(N, 32 * T)              # [n, (j t e)]
            idx[:, k0:k0 + 32 * T] |= (b << (bits - 1 - p)).astype(np.uint8)
    return idx


def pack_layer(codes: np.ndarray, luts: dict, parent_bits: int = 8) -> dict:
    """State-dict entries of one linear as the reference checkpoint names them
    (pack.py:101-112): ``qweight`` and ``lut{b}``; ``luts[b]`` is fp16 ``[N, 2**b]``."""
    N = codes.shape[0]
    entries = {"qweight": pack_codes(codes, parent_bits)}
    for b, table in sorted(luts.items()):
        table = np.ascontiguousarray(table, dtype=np.float16)
        if table.shape != (N, 1 << b):
            raise ValueError(f"lut{b} must be [{N}, {1 << b}], got {table.shape}")
        entries[f"lut{b}"] = table
    return entries

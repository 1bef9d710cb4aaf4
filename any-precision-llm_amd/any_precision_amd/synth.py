"""Seeded synthetic layers of the benchmark configurations.

Codes are uniform in ``[0, 2**parent)``; every precision ``b`` gets an
independent per-row table of ``2**b`` ascending draws from N(0, 0.02**2)
(0.02 is the standard deviation); activations are fp16 N(0, 1).
"""
from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np

from .packing import pack_codes

LLAMA2_7B_LAYER = (("q_proj", 4096, 4096), ("k_proj", 4096, 4096), ("v_proj", 4096, 4096), ("o_proj", 4096, 4096),
                   ("gate_proj", 11008, 4096), ("up_proj", 11008, 4096), ("down_proj", 4096, 11008))
LLAMA3_8B_LAYER = (("q_proj", 4096, 4096), ("k_proj", 1024, 4096), ("v_proj", 1024, 4096), ("o_proj", 4096, 4096),
                   ("gate_proj", 14336, 4096), ("up_proj", 14336, 4096), ("down_proj", 4096, 14336))


@dataclass
class SynthLayer:
    N: int
    K: int
    parent_bits: int
    seed_bits: int
    codes: np.ndarray                      # uint8 [N, K]
    qweight: np.ndarray                    # int32 [P, N, K/32]
    luts: dict = field(default_factory=dict)   # b -> fp16 [N, 2**b]


def make_luts(N: int, bits, rng: np.random.Generator, std: float = 0.02) -> dict:
    return {b: np.sort(rng.normal(0.0, std, size=(N, 1 << b)), axis=1).astype(np.float16) for b in bits}


def make_layer(N: int, K: int, seed: int = 0, parent_bits: int = 8, seed_bits: int = 3) -> SynthLayer:
    rng = np.random.default_rng(seed)
    codes = rng.integers(0, 1 << parent_bits, size=(N, K), dtype=np.uint8)
    luts = make_luts(N, range(seed_bits, parent_bits + 1), rng)
    return SynthLayer(N, K, parent_bits, seed_bits, codes, pack_codes(codes, parent_bits), luts)


def make_x(M: int, K: int, seed: int = 0) -> np.ndarray:
    return np.random.default_rng(10_000 + seed).normal(0.0, 1.0, size=(M, K)).astype(np.float16)


def gemv_bytes(N: int, K: int, w_bits: int, M: int = 1) -> int:
    """Algorithmic bytes of one GEMV call: planes + table + activations + result."""
    return w_bits * N * K // 8 + N * (1 << w_bits) * 2 + 2 * M * K + 2 * M * N


def dequant_bytes(N: int, K: int, w_bits: int) -> int:
    """Algorithmic bytes of one dequant call: planes + table + fp16 result."""
    return w_bits * N * K // 8 + N * (1 << w_bits) * 2 + 2 * N * K

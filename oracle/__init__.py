"""CPU oracle for the bitplane path -- TEST INFRASTRUCTURE ONLY.

Only the test-suite, ``__graft_entry__.smoke()`` and the CPU-baseline leg of
``bench.py`` may import this package.  The shipped library never does: it has
no CPU fallback and fails loudly when the HIP library is missing.

Two independent statements of the reference live here:

* ``libanyprec_oracle.so`` (``anyprec_oracle.c``): C restatement of the pack
  layout, the per-lane bit transpose, the dequant kernel walk and the GEMV
  kernel walk, each function citing the reference lines it follows.
* ``np_pack_bitplanes`` below: the packer as the reference's ``pack.py``
  writes it (``np.packbits`` + byte permutation by ``argsort``), in numpy.

The tests play one against the other and both against closed forms.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libanyprec_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile the C oracle with gcc (seconds)."""
    if force or not os.path.exists(_LIB_PATH) or (
        os.path.getmtime(_LIB_PATH) < os.path.getmtime(os.path.join(_HERE, "anyprec_oracle.c"))
    ):
        subprocess.check_call(["make", "-C", _HERE, "-B", "all"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        vp, ci = ctypes.c_void_p, ctypes.c_int
        L.apo_pack_bitplanes.argtypes = [vp, ci, ci, ci, vp]
        L.apo_pack_bitplanes.restype = ci
        L.apo_transpose.argtypes = [vp, ci, vp]
        L.apo_transpose.restype = None
        L.apo_transpose_pair.argtypes = [vp, ci, vp]
        L.apo_transpose_pair.restype = None
        L.apo_dequant_kbit.argtypes = [vp, ci, ci, ci, vp, vp]
        L.apo_dequant_kbit.restype = ci
        L.apo_matmul_kbit.argtypes = [vp, vp, ci, ci, ci, ci, vp, vp, vp]
        L.apo_matmul_kbit.restype = ci
        L.apo_matmul_kbit_fast.argtypes = [vp, vp, ci, ci, ci, ci, vp, vp]
        L.apo_matmul_kbit_fast.restype = ci
        L.apo_half_to_float.argtypes = [ctypes.c_uint16]
        L.apo_half_to_float.restype = ctypes.c_float
        L.apo_double_to_half.argtypes = [ctypes.c_double]
        L.apo_double_to_half.restype = ctypes.c_uint16
        L.apo_num_threads.argtypes = []
        L.apo_num_threads.restype = ci
        _lib = L
    return _lib


def _p(a: np.ndarray) -> ctypes.c_void_p:
    return ctypes.c_void_p(a.ctypes.data)


def _c(a, dtype) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=dtype)


# --------------------------------------------------------------------------
# C oracle wrappers
# --------------------------------------------------------------------------

def pack_bitplanes(codes: np.ndarray, parent_bits: int = 8) -> np.ndarray:
    """codes uint8 [N,K] -> qweight int32 [P,N,K/32] (pack.py:90-99)."""
    codes = _c(codes, np.uint8)
    N, K = codes.shape
    out = np.empty((parent_bits, N, K // 32), dtype=np.uint32)
    rc = lib().apo_pack_bitplanes(_p(codes), N, K, parent_bits, _p(out))
    if rc != 0:
        raise ValueError(f"apo_pack_bitplanes rc={rc}")
    return out.view(np.int32)


def transpose(q: np.ndarray, bits: int) -> np.ndarray:
    """One lane's plane words q[bits] -> q_w[8] (dequant.cuh dequant<bits,false>)."""
    q = _c(q, np.uint32)
    assert q.shape == (bits,)
    out = np.empty(8, dtype=np.uint32)
    lib().apo_transpose(_p(q), bits, _p(out))
    return out


def transpose_pair(q: np.ndarray, bits: int) -> np.ndarray:
    """dequant<bits,true>: q_w[4], byte = (idx(e=m) << bits) | idx(e=m+4)."""
    q = _c(q, np.uint32)
    out = np.empty(4, dtype=np.uint32)
    lib().apo_transpose_pair(_p(q), bits, _p(out))
    return out


def dequant_kbit(qweight: np.ndarray, lut: np.ndarray, w_bits: int) -> np.ndarray:
    """qweight int32 [>=b,N,K/32], lut fp16 [N,2^b] -> fp16 [N,K] (dequant.cuh:177-242)."""
    qw = _c(qweight, np.int32).view(np.uint32)
    lut = _c(lut, np.float16)
    _, N, W = qw.shape
    assert qw.shape[0] >= w_bits and lut.shape == (N, 1 << w_bits)
    out = np.empty((N, W * 32), dtype=np.float16)
    rc = lib().apo_dequant_kbit(_p(qw), N, W * 32, w_bits, _p(lut.view(np.uint16)), _p(out.view(np.uint16)))
    if rc != 0:
        raise ValueError(f"apo_dequant_kbit rc={rc}")
    return out


def matmul_kbit(x: np.ndarray, qweight: np.ndarray, lut: np.ndarray, w_bits: int, return_f64: bool = False):
    """x fp16 [...,K] -> fp16 [...,N]; double accumulate, one rounding (matmul.cuh:16-167)."""
    qw = _c(qweight, np.int32).view(np.uint32)
    lut = _c(lut, np.float16)
    x = _c(x, np.float16)
    _, N, W = qw.shape
    K = W * 32
    M = x.size // K
    assert x.shape[-1] == K and lut.shape == (N, 1 << w_bits)
    out = np.empty((M, N), dtype=np.float16)
    outd = np.empty((M, N), dtype=np.float64)
    rc = lib().apo_matmul_kbit(_p(x.view(np.uint16)), _p(qw), M, N, K, w_bits,
                               _p(lut.view(np.uint16)), _p(out.view(np.uint16)), _p(outd))
    if rc != 0:
        raise ValueError(f"apo_matmul_kbit rc={rc}")
    shape = x.shape[:-1] + (N,)
    if return_f64:
        return out.reshape(shape), outd.reshape(shape)
    return out.reshape(shape)


def matmul_kbit_fast(x: np.ndarray, qweight: np.ndarray, lut: np.ndarray, w_bits: int) -> np.ndarray:
    """Host-speed arrangement of the same semantics (fp32 accumulate, OpenMP over rows)."""
    qw = _c(qweight, np.int32).view(np.uint32)
    lut = _c(lut, np.float16)
    x = _c(x, np.float16)
    _, N, W = qw.shape
    K = W * 32
    M = x.size // K
    out = np.empty((M, N), dtype=np.float16)
    rc = lib().apo_matmul_kbit_fast(_p(x.view(np.uint16)), _p(qw), M, N, K, w_bits,
                                    _p(lut.view(np.uint16)), _p(out.view(np.uint16)))
    if rc != 0:
        raise ValueError(f"apo_matmul_kbit_fast rc={rc}")
    return out.reshape(x.shape[:-1] + (N,))


def num_threads() -> int:
    return int(lib().apo_num_threads())


# --------------------------------------------------------------------------
# numpy statement of pack.py (independent of the C packer)
# --------------------------------------------------------------------------

def _np_new_indices(byte_indices: np.ndarray, threads: int, offset: int = 0) -> np.ndarray:
    # pack.py:51-68
    bytes_per_warp = threads * 4
    warp_idx, within = np.divmod(byte_indices, bytes_per_warp)
    lane = byte_indices % threads
    in_lane = (within // threads) ^ 3
    return warp_idx * bytes_per_warp + lane * 4 + in_lane + offset


def np_pack_bitplanes(codes: np.ndarray, parent_bits: int = 8) -> np.ndarray:
    """pack.py:12-48,71-76,90-99 in numpy: packbits per plane (MSB plane first),
    byte permutation through argsort, little-endian int32 view."""
    codes = _c(codes, np.uint8)
    N, K = codes.shape
    assert K % 32 == 0
    flat = codes.reshape(-1)
    planes = np.empty((parent_bits, flat.size // 8), dtype=np.uint8)
    mask = 1 << (parent_bits - 1)
    for bit in range(parent_bits):
        planes[bit] = np.packbits((flat & mask).astype(bool))
        mask >>= 1
    planes = planes.reshape(parent_bits, N, K // 8)
    total = K // 8
    full = (total // 128) * 128
    new_idx = np.empty(total, dtype=np.int64)
    new_idx[:full] = _np_new_indices(np.arange(full), 32)
    if total - full:
        rem = np.arange(total - full)
        new_idx[full:] = _np_new_indices(rem, rem.size // 4, offset=full)
    permuted = planes[:, :, np.argsort(new_idx)]
    return np.ascontiguousarray(permuted).reshape(-1, 4).view("<i4").reshape(parent_bits, N, total // 4)

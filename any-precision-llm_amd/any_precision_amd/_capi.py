"""ctypes binding of libanyprec_hip.so (the C ABI declared in include/anyprec_hip.h).

There is no fallback: if the library is missing, importing this module raises.
"""
from __future__ import annotations

import ctypes
import os

_PKG_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB_PATH = os.path.join(_PKG_ROOT, "lib", "libanyprec_hip.so")

AP_OK = 0
AP_ENULL, AP_EBITS, AP_ESHAPE, AP_EALIGN, AP_EBATCH, AP_ELIMIT, AP_EKNOB = -1, -2, -3, -4, -5, -6, -7
AP_ABI_VERSION = 8

if not os.path.exists(LIB_PATH):
    raise ModuleNotFoundError(
        f"{LIB_PATH} is missing: build it with `python any-precision-llm_amd/build.py` "
        "(hipcc, --offload-arch=gfx950). There is no CPU fallback."
    )

lib = ctypes.CDLL(LIB_PATH)

_vp, _ci = ctypes.c_void_p, ctypes.c_int
lib.ap_abi_version.argtypes = []
lib.ap_abi_version.restype = _ci
lib.ap_strerror.argtypes = [_ci]
lib.ap_strerror.restype = ctypes.c_char_p
lib.ap_dequant_kbit.argtypes = [_vp, _vp, _vp, _ci, _ci, _ci, _vp]
lib.ap_dequant_kbit.restype = _ci
lib.ap_matmul_kbit.argtypes = [_vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci, _vp]
lib.ap_matmul_kbit.restype = _ci
lib.ap_gemm_kbit.argtypes = [_vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci, _vp]
lib.ap_gemm_kbit.restype = _ci
_pi = ctypes.POINTER(ctypes.c_int)
_pvp = ctypes.POINTER(ctypes.c_void_p)
lib.ap_dequant_kbit_group.argtypes = [_ci, _pvp, _pvp, _pvp, _pi, _pi, _ci, _vp]
lib.ap_dequant_kbit_group.restype = _ci
lib.ap_gemm_kbit_pays.argtypes = [_ci, _ci, _ci, _ci]
lib.ap_gemm_kbit_pays.restype = _ci
lib.ap_gemm_kbit_group_pays.argtypes = [_ci, _pi, _ci, _ci, _ci]
lib.ap_gemm_kbit_group_pays.restype = _ci
lib.ap_matmul_kbit_group.argtypes = [_vp, _ci, _pvp, _pvp, _pvp, _pi, _ci, _ci, _ci, _vp]
lib.ap_matmul_kbit_group.restype = _ci
_pll = ctypes.POINTER(ctypes.c_longlong)
lib.ap_gemm_kbit_group.argtypes = [_vp, _ci, _pvp, _pvp, _pvp, _pi, _pll, _ci, _ci, _ci, _vp]
lib.ap_gemm_kbit_group.restype = _ci
lib.ap_matmul_kbit_geometry.argtypes = [_ci, _ci, _ci, _ci, _pi, _pi, _pi, _pi]
lib.ap_matmul_kbit_geometry.restype = _ci
lib.ap_probe_stream.argtypes = [_vp, ctypes.c_longlong, _vp, ctypes.c_longlong, _vp, _ci, _vp]
lib.ap_probe_stream.restype = _ci
lib.ap_probe_write.argtypes = [_vp, ctypes.c_longlong, ctypes.c_uint32, _ci, _vp]
lib.ap_probe_write.restype = _ci
lib.ap_probe_empty.argtypes = [_vp, _vp]
lib.ap_probe_empty.restype = _ci
lib.ap_matmul_kbit_route.argtypes = [_ci, _ci, _ci, _ci, _pi]
lib.ap_matmul_kbit_route.restype = _ci
lib.ap_matmul_kbit_group_route.argtypes = [_ci, _pi, _ci, _ci, _ci, _pi, _pi]
lib.ap_matmul_kbit_group_route.restype = _ci
lib.ap_matmul_kbit_swiglu.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci, _vp]
lib.ap_matmul_kbit_swiglu.restype = _ci
lib.ap_add_rmsnorm.argtypes = [_vp, _vp, _vp, _vp, _vp, _ci, _ci, ctypes.c_float, _vp]
lib.ap_add_rmsnorm.restype = _ci
lib.ap_silu_mul.argtypes = [_vp, _vp, _vp, ctypes.c_longlong, _vp]
lib.ap_silu_mul.restype = _ci
lib.ap_decode_attention.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci, ctypes.c_float, _vp]
lib.ap_decode_attention.restype = _ci
lib.ap_decode_advance.argtypes = [_vp, _ci, _vp, _vp, _vp, _ci, _vp]
lib.ap_decode_advance.restype = _ci
lib.ap_set_tuning.argtypes = [ctypes.c_char_p, _ci]
lib.ap_set_tuning.restype = _ci
lib.ap_get_tuning.argtypes = [ctypes.c_char_p, _pi]
lib.ap_get_tuning.restype = _ci

if lib.ap_abi_version() != AP_ABI_VERSION:
    raise ImportError(
        f"{LIB_PATH} has ABI version {lib.ap_abi_version()}, this binding needs {AP_ABI_VERSION}: rebuild it"
    )

EXPORTS = ("ap_abi_version", "ap_strerror", "ap_dequant_kbit", "ap_matmul_kbit", "ap_matmul_kbit_group",
           "ap_gemm_kbit", "ap_matmul_kbit_geometry", "ap_set_tuning", "ap_get_tuning", "ap_probe_stream", "ap_probe_empty", "ap_probe_write", "ap_matmul_kbit_route", "ap_matmul_kbit_group_route",
           "ap_add_rmsnorm", "ap_silu_mul", "ap_decode_attention", "ap_matmul_kbit_swiglu", "ap_decode_advance", "ap_gemm_kbit_group", "ap_dequant_kbit_group", "ap_gemm_kbit_pays",
           "ap_gemm_kbit_group_pays")
GEMM_MAX_M = 128
GROUP_MAX = 4
DEQUANT_GROUP_MAX = 8


def dequant_group(qweights, luts, outs, rows, cols, w_bits: int, stream: int) -> int:
    """ap_dequant_kbit_group on raw device addresses (lists of equal length <= DEQUANT_GROUP_MAX)."""
    n = len(qweights)
    arr = ctypes.c_void_p * n
    ints = ctypes.c_int * n
    return lib.ap_dequant_kbit_group(n, arr(*qweights), arr(*luts), arr(*outs), ints(*rows), ints(*cols), w_bits, stream)


def gemm_pays(M: int, N: int, K: int, w_bits: int) -> bool:
    """ap_gemm_kbit_pays: the fused GEMM beats dequant_kbit + a library GEMM for this shape."""
    rc = lib.ap_gemm_kbit_pays(M, N, K, w_bits)
    if rc < 0:
        check(rc, "ap_gemm_kbit_pays")
    return rc == 1


def gemm_group_pays(M: int, rows, K: int, w_bits: int) -> bool:
    """ap_gemm_kbit_group_pays: one tiled launch over the set beats its members one by one."""
    n = len(rows)
    if not 1 <= n <= GROUP_MAX:
        return False
    rc = lib.ap_gemm_kbit_group_pays(n, (ctypes.c_int * n)(*rows), M, K, w_bits)
    if rc < 0:
        check(rc, "ap_gemm_kbit_group_pays")
    return rc == 1


def matmul_group(x_ptr: int, qweights, luts, outs, rows, M: int, K: int, w_bits: int, stream: int) -> int:
    """ap_matmul_kbit_group on raw device addresses (lists of equal length <= GROUP_MAX)."""
    n = len(qweights)
    arr = ctypes.c_void_p * n
    return lib.ap_matmul_kbit_group(x_ptr, n, arr(*qweights), arr(*luts), arr(*outs), (ctypes.c_int * n)(*rows),
                                    M, K, w_bits, stream)


def gemm_group(x_ptr: int, qweights, luts, outs, rows, ldo, M: int, K: int, w_bits: int, stream: int) -> int:
    """ap_gemm_kbit_group on raw device addresses (lists of equal length <= GROUP_MAX; ldo: row strides or None)."""
    n = len(qweights)
    arr = ctypes.c_void_p * n
    strides = None if ldo is None else (ctypes.c_longlong * n)(*ldo)
    return lib.ap_gemm_kbit_group(x_ptr, n, arr(*qweights), arr(*luts), arr(*outs), (ctypes.c_int * n)(*rows), strides,
                                  M, K, w_bits, stream)


def strerror(code: int) -> str:
    return lib.ap_strerror(code).decode()


def check(code: int, what: str) -> None:
    """Argument errors -> ValueError, HIP launch errors -> RuntimeError."""
    if code == AP_OK:
        return
    if code < 0:
        raise ValueError(f"{what}: {strerror(code)} (code {code})")
    raise RuntimeError(f"{what}: HIP error {code}: {strerror(code)}")


def matmul_geometry(M: int, N: int, K: int, w_bits: int) -> dict:
    vals = [ctypes.c_int() for _ in range(4)]
    check(lib.ap_matmul_kbit_geometry(M, N, K, w_bits, *[ctypes.byref(v) for v in vals]), "ap_matmul_kbit_geometry")
    return dict(zip(("wpl", "segments", "rows", "grid"), (v.value for v in vals)))


ROUTES = ("dot", "stream", "fine", "mfma4", "mfma16")


def matmul_route(M: int, N: int, K: int, w_bits: int) -> str:
    """Name of the kernel ap_matmul_kbit launches for one linear of this shape."""
    r = ctypes.c_int()
    check(lib.ap_matmul_kbit_route(M, N, K, w_bits, ctypes.byref(r)), "ap_matmul_kbit_route")
    return ROUTES[r.value]


def matmul_group_route(M: int, rows, K: int, w_bits: int):
    """(kernel name per member, weight rows per workgroup of the joint dot-product launch) for a set of linears."""
    n = len(rows)
    r = (ctypes.c_int * n)()
    per_wg = ctypes.c_int()
    check(lib.ap_matmul_kbit_group_route(n, (ctypes.c_int * n)(*rows), M, K, w_bits, r, ctypes.byref(per_wg)),
          "ap_matmul_kbit_group_route")
    return [ROUTES[v] for v in r], per_wg.value


def set_tuning(name: str, value: int) -> None:
    """ap_set_tuning: override one launch-heuristic knob for this process (tests, benchmarks)."""
    check(lib.ap_set_tuning(name.encode(), int(value)), f"ap_set_tuning({name})")


def get_tuning(name: str) -> int:
    val = ctypes.c_int()
    check(lib.ap_get_tuning(name.encode(), ctypes.byref(val)), f"ap_get_tuning({name})")
    return val.value


class tuning:
    """Context manager: `with tuning(gemm_rb2=2): ...` sets knobs and restores them on exit."""

    def __init__(self, **knobs):
        self.knobs = knobs
        self.saved = {}

    def __enter__(self):
        for k, v in self.knobs.items():
            self.saved[k] = get_tuning(k)
            set_tuning(k, v)
        return self

    def __exit__(self, *exc):
        for k, v in self.saved.items():
            set_tuning(k, v)
        return False

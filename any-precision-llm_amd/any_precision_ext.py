"""Drop-in replacement for the reference's native module ``any_precision_ext``
(any_precision/modules/kernels/main.cu:145-148): same op names, same positional
signatures, same result shapes and dtypes.

    matmul_kbit(in, qweight, lut, w_bits) -> Tensor   main.cu:93-143
    dequant_kbit(qweight, lut, w_bits)    -> Tensor   main.cu:60-91

plus one op the reference does not have, ``gemm_kbit(in, qweight, lut, w_bits)``: the
fused dequant -> MFMA GEMM (the reference's ``dequant_kbit`` + ``torch.matmul`` branch,
AnyPrecisionLinear.py:60-62, in one launch per ``GEMM_MAX_M`` activation rows).

The ops validate their arguments, allocate the result with torch and hand raw
device pointers plus torch's current HIP stream to libanyprec_hip.so.  Where
the reference asserts (compiled out in release builds) or exits the process,
these raise ``ValueError`` / ``RuntimeError``.  Launches go to the *current*
stream (the reference uses the legacy default stream, main.cu:83,134), so the
ops can be captured into HIP graphs.
"""
from __future__ import annotations

import torch

from any_precision_amd import _capi

__all__ = ["matmul_kbit", "dequant_kbit", "dequant_kbit_group", "gemm_kbit", "gemm_kbit_group", "matmul_kbit_group", "matmul_kbit_swiglu", "GEMM_MAX_M"]

GEMM_MAX_M = _capi.GEMM_MAX_M

_lib = _capi.lib


def _check_weight(qweight: torch.Tensor, lut: torch.Tensor, w_bits: int, op: str):
    if not isinstance(w_bits, int) or isinstance(w_bits, bool):
        raise TypeError(f"{op}: w_bits must be an int, got {type(w_bits).__name__}")
    if w_bits < 3 or w_bits > 8:
        raise ValueError(f"{op}: w_bits must be in 3..8, got {w_bits}")
    if qweight.dim() != 3 or qweight.dtype != torch.int32:
        raise ValueError(f"{op}: qweight must be a 3-D int32 tensor [planes, N, K/32], got "
                         f"{tuple(qweight.shape)} {qweight.dtype}")
    if lut.dtype != torch.float16:
        raise ValueError(f"{op}: lut must be float16, got {lut.dtype}")
    if not qweight.is_cuda or qweight.device != lut.device:
        raise ValueError(f"{op}: qweight and lut must live on the same GPU, got {qweight.device} and {lut.device}")
    planes, N, W = qweight.shape
    if planes < w_bits:
        raise ValueError(f"{op}: qweight holds {planes} planes, w_bits={w_bits} needs {w_bits}")
    if N < 1 or W < 1:
        raise ValueError(f"{op}: empty weight {tuple(qweight.shape)}")
    if tuple(lut.shape) != (N, 1 << w_bits):
        raise ValueError(f"{op}: lut must be [{N}, {1 << w_bits}] for w_bits={w_bits}, got {tuple(lut.shape)}")
    if not qweight.is_contiguous() or not lut.is_contiguous():
        raise ValueError(f"{op}: qweight and lut must be contiguous")
    return N, W * 32


def dequant_kbit(qweight: torch.Tensor, lut: torch.Tensor, w_bits: int) -> torch.Tensor:
    """fp16 [N, K] with out[n, k] = lut[n, code[n, k] >> (P - w_bits)]."""
    N, K = _check_weight(qweight, lut, w_bits, "dequant_kbit")
    with torch.cuda.device(qweight.device):
        out = torch.empty((N, K), dtype=torch.float16, device=qweight.device)
        rc = _lib.ap_dequant_kbit(qweight.data_ptr(), lut.data_ptr(), out.data_ptr(), N, K, w_bits,
                                  torch.cuda.current_stream().cuda_stream)
    _capi.check(rc, "dequant_kbit")
    return out


def dequant_kbit_group(qweights, luts, w_bits: int):
    """``[dequant_kbit(q, t, w_bits) for q, t in zip(qweights, luts)]`` in ONE launch: up to DEQUANT_GROUP_MAX linears of
    any shapes on one GPU at one bit-width (a decoder layer has seven).  No counterpart in the reference, which launches
    its kernel once per linear (main.cu:82-84); results are bit-identical to the separate calls."""
    if len(qweights) != len(luts) or not 1 <= len(qweights) <= _capi.DEQUANT_GROUP_MAX:
        raise ValueError(f"dequant_kbit_group: need 1..{_capi.DEQUANT_GROUP_MAX} (qweight, lut) pairs")
    shapes = [_check_weight(q, t, w_bits, "dequant_kbit_group") for q, t in zip(qweights, luts)]
    dev = qweights[0].device
    if any(q.device != dev for q in qweights):
        raise ValueError("dequant_kbit_group: all weights must be on one device")
    with torch.cuda.device(dev):
        outs = [torch.empty((N, K), dtype=torch.float16, device=dev) for N, K in shapes]
        rc = _capi.dequant_group([q.data_ptr() for q in qweights], [t.data_ptr() for t in luts], [o.data_ptr() for o in outs],
                                 [N for N, _ in shapes], [K for _, K in shapes], w_bits, torch.cuda.current_stream().cuda_stream)
    _capi.check(rc, "dequant_kbit_group")
    return outs


def matmul_kbit(in_: torch.Tensor, qweight: torch.Tensor, lut: torch.Tensor, w_bits: int) -> torch.Tensor:
    """fp16 in_.shape[:-1] + [N]; M = in_.numel() // K must be in 1..8 (main.cu:108)."""
    N, K = _check_weight(qweight, lut, w_bits, "matmul_kbit")
    if in_.dtype != torch.float16:
        raise ValueError(f"matmul_kbit: input must be float16, got {in_.dtype}")
    if in_.device != qweight.device:
        raise ValueError(f"matmul_kbit: input on {in_.device}, weight on {qweight.device}")
    if in_.dim() < 1 or in_.shape[-1] != K:
        raise ValueError(f"matmul_kbit: input last dim must be K={K}, got {tuple(in_.shape)}")
    M = in_.numel() // K
    if M < 1 or M > 8:
        raise ValueError(f"matmul_kbit: batch M={M} outside 1..8; use dequant_kbit + matmul for larger batches")
    if not in_.is_contiguous():
        raise ValueError("matmul_kbit: input must be contiguous")
    with torch.cuda.device(qweight.device):
        out = torch.empty(in_.shape[:-1] + (N,), dtype=torch.float16, device=in_.device)
        rc = _lib.ap_matmul_kbit(in_.data_ptr(), qweight.data_ptr(), lut.data_ptr(), out.data_ptr(), M, N, K,
                                 w_bits, torch.cuda.current_stream().cuda_stream)
    _capi.check(rc, "matmul_kbit")
    return out


def matmul_kbit_group(in_: torch.Tensor, qweights, luts, w_bits: int, concat: bool = False):
    """``[matmul_kbit(in_, q, t, w_bits) for q, t in zip(qweights, luts)]`` in one launch: up to
    GROUP_MAX linears that share the input and the bit-width (q/k/v, gate/up).  No counterpart in
    the reference; results equal the separate calls bit for bit.  ``concat=True`` returns the
    results joined along the last dimension as one tensor (for a single activation row they are
    written side by side into one allocation; otherwise joined with ``torch.cat``)."""
    if len(qweights) != len(luts) or not 1 <= len(qweights) <= _capi.GROUP_MAX:
        raise ValueError(f"matmul_kbit_group: need 1..{_capi.GROUP_MAX} (qweight, lut) pairs")
    shapes = [_check_weight(q, t, w_bits, "matmul_kbit_group") for q, t in zip(qweights, luts)]
    K = shapes[0][1]
    if any(k != K for _, k in shapes):
        raise ValueError("matmul_kbit_group: all members must have the same in_features")
    if in_.dtype != torch.float16:
        raise ValueError(f"matmul_kbit_group: input must be float16, got {in_.dtype}")
    if any(q.device != in_.device for q in qweights):
        raise ValueError("matmul_kbit_group: input and weights must be on one device")
    if in_.dim() < 1 or in_.shape[-1] != K:
        raise ValueError(f"matmul_kbit_group: input last dim must be K={K}, got {tuple(in_.shape)}")
    M = in_.numel() // K
    if M < 1 or M > 8:
        raise ValueError(f"matmul_kbit_group: batch M={M} outside 1..8")
    if not in_.is_contiguous():
        raise ValueError("matmul_kbit_group: input must be contiguous")
    with torch.cuda.device(in_.device):
        joint = None
        if concat and M == 1:
            joint = torch.empty(in_.shape[:-1] + (sum(N for N, _ in shapes),), dtype=torch.float16, device=in_.device)
            outs = list(torch.split(joint, [N for N, _ in shapes], dim=-1))       # one row: every part is dense
        else:
            outs = [torch.empty(in_.shape[:-1] + (N,), dtype=torch.float16, device=in_.device) for N, _ in shapes]
        rc = _capi.matmul_group(in_.data_ptr(), [q.data_ptr() for q in qweights], [t.data_ptr() for t in luts],
                                [o.data_ptr() for o in outs], [N for N, _ in shapes], M, K, w_bits,
                                torch.cuda.current_stream().cuda_stream)
    _capi.check(rc, "matmul_kbit_group")
    if concat:
        return joint if joint is not None else torch.cat(outs, dim=-1)
    return outs


def gemm_kbit_group(in_: torch.Tensor, qweights, luts, w_bits: int, concat: bool = False):
    """``[gemm_kbit(in_, q, t, w_bits) for q, t in zip(qweights, luts)]`` for up to GROUP_MAX linears that share the
    input and the bit-width, any number of activation rows: ONE launch of the tiled kernel where it serves the set
    (rows of a multiple of 128 elements) and pays, a launch per member otherwise.  ``concat=True`` returns the results
    joined along the last dimension as one tensor (written side by side into one allocation where the tiled kernel
    serves the set; joined with ``torch.cat`` otherwise).  No counterpart in the reference."""
    if len(qweights) != len(luts) or not 1 <= len(qweights) <= _capi.GROUP_MAX:
        raise ValueError(f"gemm_kbit_group: need 1..{_capi.GROUP_MAX} (qweight, lut) pairs")
    shapes = [_check_weight(q, t, w_bits, "gemm_kbit_group") for q, t in zip(qweights, luts)]
    K = shapes[0][1]
    if any(k != K for _, k in shapes):
        raise ValueError("gemm_kbit_group: all members must have the same in_features")
    if in_.dtype != torch.float16:
        raise ValueError(f"gemm_kbit_group: input must be float16, got {in_.dtype}")
    if any(q.device != in_.device for q in qweights):
        raise ValueError("gemm_kbit_group: input and weights must be on one device")
    if in_.dim() < 1 or in_.shape[-1] != K:
        raise ValueError(f"gemm_kbit_group: input last dim must be K={K}, got {tuple(in_.shape)}")
    M = in_.numel() // K if K else 0
    if M < 1:
        raise ValueError("gemm_kbit_group: empty input")
    if not in_.is_contiguous():
        raise ValueError("gemm_kbit_group: input must be contiguous")
    rows = [N for N, _ in shapes]
    with torch.cuda.device(in_.device):
        joint, ldo = None, None
        if concat and K % 128 == 0:      # the tiled kernel writes rows that are not dense
            joint = torch.empty(in_.shape[:-1] + (sum(rows),), dtype=torch.float16, device=in_.device)
            outs = list(torch.split(joint, rows, dim=-1))
            ldo = [sum(rows)] * len(rows)
        else:
            outs = [torch.empty(in_.shape[:-1] + (N,), dtype=torch.float16, device=in_.device) for N in rows]
        rc = _capi.gemm_group(in_.data_ptr(), [q.data_ptr() for q in qweights], [t.data_ptr() for t in luts],
                              [o.data_ptr() for o in outs], rows, ldo, M, K, w_bits, torch.cuda.current_stream().cuda_stream)
        if rc == _capi.AP_ELIMIT and joint is not None:
            # beyond the tiled kernel's geometry (it alone writes side by side): dense results, joined below
            joint = None
            outs = [torch.empty(in_.shape[:-1] + (N,), dtype=torch.float16, device=in_.device) for N in rows]
            rc = _capi.gemm_group(in_.data_ptr(), [q.data_ptr() for q in qweights], [t.data_ptr() for t in luts],
                                  [o.data_ptr() for o in outs], rows, None, M, K, w_bits, torch.cuda.current_stream().cuda_stream)
    _capi.check(rc, "gemm_kbit_group")
    if concat:
        return joint if joint is not None else torch.cat(outs, dim=-1)
    return outs


def matmul_kbit_swiglu(in_: torch.Tensor, qweight_gate, lut_gate, qweight_up, lut_up, w_bits: int, out=None) -> torch.Tensor:
    """``silu(matmul_kbit(in_, gate)) * matmul_kbit(in_, up)`` for 1..4 activation rows in one launch, fp32 until the
    store.  No counterpart in the reference (its ``fuse_layers`` hook is a stub, AnyPrecisionForCausalLM.py:168-172)."""
    N, K = _check_weight(qweight_gate, lut_gate, w_bits, "matmul_kbit_swiglu")
    if _check_weight(qweight_up, lut_up, w_bits, "matmul_kbit_swiglu") != (N, K):
        raise ValueError("matmul_kbit_swiglu: gate and up must have one shape")
    if in_.dtype != torch.float16 or not in_.is_contiguous():
        raise ValueError("matmul_kbit_swiglu: input must be contiguous float16")
    if in_.device != qweight_gate.device or in_.device != qweight_up.device:
        raise ValueError("matmul_kbit_swiglu: input and weights must be on one device")
    if in_.dim() < 1 or in_.shape[-1] != K:
        raise ValueError(f"matmul_kbit_swiglu: input last dim must be K={K}, got {tuple(in_.shape)}")
    M = in_.numel() // K
    if M < 1 or M > 4:
        raise ValueError(f"matmul_kbit_swiglu: batch M={M} outside 1..4")
    with torch.cuda.device(in_.device):
        if out is None:
            out = torch.empty(in_.shape[:-1] + (N,), dtype=torch.float16, device=in_.device)
        elif out.dtype != torch.float16 or not out.is_contiguous() or out.numel() != M * N or out.device != in_.device:
            raise ValueError("matmul_kbit_swiglu: out must be a contiguous float16 tensor of M x N elements on the input's device")
        rc = _lib.ap_matmul_kbit_swiglu(in_.data_ptr(), qweight_gate.data_ptr(), lut_gate.data_ptr(), qweight_up.data_ptr(),
                                        lut_up.data_ptr(), out.data_ptr(), M, N, K, w_bits,
                                        torch.cuda.current_stream().cuda_stream)
    _capi.check(rc, "matmul_kbit_swiglu")
    return out


def gemm_kbit(in_: torch.Tensor, qweight: torch.Tensor, lut: torch.Tensor, w_bits: int) -> torch.Tensor:
    """fp16 in_.shape[:-1] + [N] = in_ @ dequant(qweight, lut, w_bits).T without materialising the fp16
    weight; one launch per GEMM_MAX_M rows."""
    N, K = _check_weight(qweight, lut, w_bits, "gemm_kbit")
    if in_.dtype != torch.float16:
        raise ValueError(f"gemm_kbit: input must be float16, got {in_.dtype}")
    if in_.device != qweight.device:
        raise ValueError(f"gemm_kbit: input on {in_.device}, weight on {qweight.device}")
    if in_.dim() < 1 or in_.shape[-1] != K:
        raise ValueError(f"gemm_kbit: input last dim must be K={K}, got {tuple(in_.shape)}")
    M = in_.numel() // K
    if M < 1:
        raise ValueError("gemm_kbit: empty batch")
    if not in_.is_contiguous():
        raise ValueError("gemm_kbit: input must be contiguous")
    with torch.cuda.device(qweight.device):
        out = torch.empty(in_.shape[:-1] + (N,), dtype=torch.float16, device=in_.device)
        rc = _lib.ap_gemm_kbit(in_.data_ptr(), qweight.data_ptr(), lut.data_ptr(), out.data_ptr(), M, N, K,
                               w_bits, torch.cuda.current_stream().cuda_stream)
    _capi.check(rc, "gemm_kbit")
    return out

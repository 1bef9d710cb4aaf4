"""``AnyPrecisionLinear``: counterpart of the reference operator module
(any_precision/modules/AnyPrecisionLinear.py:10-78) on top of the HIP ops.

Same constructor, buffers (``qweight`` int32 ``[max(supported_bits), out, in/32]``,
``lut{b}`` fp16 ``[out, 2**b]``, optional ``bias`` buffer), state-dict keys,
``forward(x, precision=...)``, ``set_precision`` and ``prune_precisions``.
Batch dispatch: up to 8 activation rows -> ``matmul_kbit`` as in the reference (:60-64);
9 .. 32 rows (up to 64, 128, 256 or 512 where the library's ``ap_gemm_kbit_pays`` says so) -> the fused
``gemm_kbit``; beyond -> ``dequant_kbit`` + ``torch.matmul`` as in the reference.
"""
from __future__ import annotations

import torch
import torch.nn as nn

try:
    from any_precision_ext import (matmul_kbit, matmul_kbit_group, matmul_kbit_swiglu, dequant_kbit, gemm_kbit, gemm_kbit_group,
                                   GEMM_MAX_M)
    from . import _capi
except ModuleNotFoundError:
    matmul_kbit, matmul_kbit_group, matmul_kbit_swiglu, dequant_kbit, gemm_kbit, gemm_kbit_group, GEMM_MAX_M = (None,) * 6 + (0,)
    _capi = None


def fused_gemm_pays(rows: int, out_features: int, w_bits: int, in_features: int) -> bool:
    """Whether the fused GEMM beats ``dequant_kbit`` + ``torch.matmul`` for ``rows`` activation rows: the library's own
    measured crossovers (``ap_gemm_kbit_pays``; the thresholds live in one place, beside the kernels' launch rules)."""
    return _capi.gemm_pays(rows, out_features, in_features, w_bits)


def fused_set_pays(rows: int, out_features, w_bits: int, in_features: int) -> bool:
    """Whether ONE launch of the tiled GEMM over linears that share their input (``gemm_kbit_group``) beats calling them
    one by one (``ap_gemm_kbit_group_pays``)."""
    return _capi.gemm_group_pays(rows, list(out_features), in_features, w_bits)


def forward_group(modules, x, precision=None, concat=False):
    """``[m(x, precision=precision) for m in modules]`` for linears that share their input (the
    q/k/v or gate/up projections of a decoder layer); with ``concat`` the results joined along
    the last dimension.  Up to 8 activation rows and 4 modules they go through ``matmul_kbit_group``, which
    issues ONE launch wherever the dot-product kernel serves the set (always up to 4 rows; at 5..8 rows for
    sets with narrow members and some 5-8-bit cases) and a launch per member otherwise; beyond 8 rows through
    ``gemm_kbit_group`` (one launch of the tiled GEMM) where the fused form pays for the set; else module by module.
    The reference has no counterpart (its ``fuse_layers`` is a stub, AnyPrecisionForCausalLM.py:168-172)."""
    rows = x.numel() // x.shape[-1]
    w_bits = modules[0].precision if precision is None else precision
    x = x.contiguous()
    K = modules[0].in_features
    same_input = 2 <= len(modules) <= 4 and all(m.in_features == K for m in modules)
    # one launch of the tiled GEMM (three 4096 x 4096 projections at 128 rows fill the chip that one of them leaves half
    # idle); up to 32 rows on wide members the K-split kernel, module by module, is as fast or faster
    tiled_set = same_input and fused_set_pays(rows, [m.out_features for m in modules], w_bits, K)
    if not same_input or (rows > 8 and not tiled_set):
        outs = [m(x, precision=w_bits) for m in modules]
        return torch.cat(outs, dim=-1) if concat else outs
    has_bias = any(m.bias is not None for m in modules)
    group_op = gemm_kbit_group if rows > 8 else matmul_kbit_group
    res = group_op(x, [m.qweight for m in modules], [m._buffers[f"lut{w_bits}"] for m in modules], w_bits,
                   concat=concat and not has_bias)
    if not has_bias:
        return res
    for m, o in zip(modules, res):
        if m.bias is not None:
            o += m.bias
    return torch.cat(res, dim=-1) if concat else res


def forward_swiglu(gate, up, x, precision=None, out=None):
    """``silu(gate(x)) * up(x)`` for two bias-free linears of one shape: up to 4 activation rows (and rows of at most
    32768 elements) in ONE launch with the activation applied before the store; otherwise the two GEMVs (one grouped
    launch where possible) and the product in PyTorch ops."""
    rows = x.numel() // x.shape[-1]
    w_bits = gate.precision if precision is None else precision
    fits = (rows <= 4 and gate.bias is None and up.bias is None and gate.in_features <= 32768
            and (gate.in_features, gate.out_features) == (up.in_features, up.out_features))
    if fits:
        return matmul_kbit_swiglu(x.contiguous(), gate.qweight, gate._buffers[f"lut{w_bits}"], up.qweight,
                                  up._buffers[f"lut{w_bits}"], w_bits, out=out)
    g, u = forward_group((gate, up), x, w_bits)
    res = torch.nn.functional.silu(g) * u
    if out is not None:
        out.copy_(res.view_as(out))
        return out
    return res


class AnyPrecisionLinear(nn.Module):
    """One bitplane-packed linear layer serving every precision in ``precisions``.

    Interface of the reference module (AnyPrecisionLinear.py:10-78): constructor arguments, the
    ``qweight`` / ``lut{b}`` / ``bias`` buffers and hence the state-dict keys, ``forward(x,
    precision=b)``, ``set_precision``, ``prune_precisions``, and the messages of its errors."""

    def __init__(self, in_features, out_features, supported_bits, bias=True, precisions=None, device=None,
                 dtype=None):
        super().__init__()
        if matmul_kbit is None or dequant_kbit is None:
            raise ModuleNotFoundError("libanyprec_hip.so is not built: run `python any-precision-llm_amd/build.py`.")
        precisions = supported_bits if precisions is None else precisions
        self._validate(in_features, precisions, dtype)
        self.in_features, self.out_features = in_features, out_features
        self.supported_bits = supported_bits
        self.precisions = precisions
        self.precision = max(precisions)          # AnyPrecisionLinear.py:26: the widest by default
        # plane p of the parent code is qweight[p] (plane 0 = most significant bit): [P, N, K/32] int32
        planes = torch.empty((max(supported_bits), out_features, in_features // 32), dtype=torch.int32, device=device)
        self.register_buffer("qweight", planes)
        # one table of 2**b centroids per row and supported bit-width
        for b in supported_bits:
            self.register_buffer(f"lut{b}", torch.empty((out_features, 1 << b), dtype=dtype, device=device))
        # a buffer, not a parameter, as in the reference (:40-46): it is loaded, never trained
        if bias:
            self.register_buffer("bias", torch.empty((out_features,), dtype=dtype, device=device))
        else:
            self.bias = None

    @staticmethod
    def _validate(in_features, precisions, dtype):
        if not isinstance(precisions, list):
            raise RuntimeError("supported_bits must be a list of integers.")
        if dtype not in (None, torch.float16):
            raise RuntimeError("Only float16 is supported for now.")
        if in_features % 32:
            raise RuntimeError("in_features must be a multiple of 32.")

    def prune_precisions(self):
        """Drops what no precision in ``precisions`` reads: planes below the widest one kept and the
        tables of the other bit-widths (AnyPrecisionLinear.py:48-52)."""
        self.qweight = self.qweight[:max(self.precisions)]
        for b in set(self.supported_bits) - set(self.precisions):
            delattr(self, f"lut{b}")

    def forward(self, x, **kwargs):
        w_bits = kwargs.get("precision", self.precision)
        table = self._buffers[f"lut{w_bits}"]
        rows = x.numel() // x.shape[-1]
        if rows <= 8:                                       # GEMV / skinny kernels (reference: :63-64)
            # the ops take dense row-major activations; a transposed or sliced view is copied (a no-op otherwise)
            y = matmul_kbit(x.contiguous(), self.qweight, table, w_bits)
        elif fused_gemm_pays(rows, self.out_features, w_bits, self.in_features):
            y = gemm_kbit(x.contiguous(), self.qweight, table, w_bits)   # fused dequant -> MFMA, weight never materialised
        else:                                               # reference: :60-62
            y = torch.matmul(x, dequant_kbit(self.qweight, table, w_bits).T)
        if self.bias is not None:
            y += self.bias
        return y

    def set_precision(self, precision):
        if precision not in self.precisions:
            raise RuntimeError(f"{self.precisions}-bit precisions are supported but {precision}-bit was specified.")
        self.precision = precision

    def extra_repr(self) -> str:
        return (f"in_features={self.in_features}, out_features={self.out_features}, bias={self.bias is not None}, "
                f"precisions={self.precisions}")

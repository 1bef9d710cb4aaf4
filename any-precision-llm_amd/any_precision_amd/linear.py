"""``AnyPrecisionLinear``: counterpart of the reference operator module
(any_precision/modules/AnyPrecisionLinear.py:10-78) on top of the HIP ops.

Same constructor, buffers (``qweight`` int32 ``[max(supported_bits), out, in/32]``,
``lut{b}`` fp16 ``[out, 2**b]``, optional ``bias`` buffer), state-dict keys,
``forward(x, precision=...)``, ``set_precision`` and ``prune_precisions``.
Batch dispatch: up to 8 activation rows -> ``matmul_kbit`` as in the reference (:60-64);
9 .. 32 rows (.. 64, 128 or 256 where ``fused_gemm_pays`` says so) -> the fused ``gemm_kbit``; beyond ->
``dequant_kbit`` + ``torch.matmul`` as in the reference.
"""
from __future__ import annotations

import torch
import torch.nn as nn

try:
    from any_precision_ext import (matmul_kbit, matmul_kbit_group, matmul_kbit_swiglu, dequant_kbit, gemm_kbit, gemm_kbit_group,
                                   GEMM_MAX_M)
except ModuleNotFoundError:
    matmul_kbit, matmul_kbit_group, matmul_kbit_swiglu, dequant_kbit, gemm_kbit, gemm_kbit_group, GEMM_MAX_M = (None,) * 6 + (0,)


def fused_gemm_pays(rows: int, out_features: int, w_bits: int, in_features: int = 0) -> bool:
    """Whether the fused GEMM beats dequant_kbit + torch.matmul.  Measured on the linear shapes of the Llama-2-7B /
    Llama-3-8B / 13B / 70B layers at 96..512 activation rows and every bit-width (fused / pair, us):

    * always up to 32 activation rows (1.3-4x at 16);
    * rows of a multiple of 128 elements (the tiled kernel), linears of at least 4096 rows: up to 128 activation rows
      at every bit-width (11008 x 4096, 8 bits: 50 / 58; 28672 x 8192: 189 / 234; 5120 x 13824: 93 / 113); up to 256
      at up to 5 bits (11008 x 4096, 4 bits: 58 / 73; 13824 x 5120, 5 bits: 79 / 97), at 6 bits except on linears of
      more than 16384 rows (28672 x 8192: 263 / 250), at 7 and 8 bits on linears of at most 8192 rows
      (8192 x 8192, 8 bits: 87 / 116; 5120 x 5120: 56 / 69; 4096 x 11008: 82 / 82; 11008 x 4096: 96 / 66); up to 512 at
      3 bits on linears of at most 8192 rows (4096 x 11008: 87 / 99; 8192 x 8192: 101 / 114; 14336 x 4096: 99 / 90);
    * the same rows on linears of 1024..4095 rows: up to 512 activation rows at 3 and 4 bits (1024 x 4096: 11-15 /
      18-23; at 6 bits and more the pair wins);
    * other row lengths (the K-split kernel only): up to 64 on linears of fewer than 8192 rows, and on larger ones at up
      to 5 bits -- except, on rows of more than 4096 elements, from 6 bits on linears of 5120 rows or more and from 5
      bits on linears of at most 2048 rows; up to 128 on linears of 4096..8191 rows of at most 4096 elements.

    Beyond, one table lookup per weight and tile of activation rows costs more than materialising the weight once."""
    if rows <= min(32, GEMM_MAX_M):
        return True
    if GEMM_MAX_M and in_features > 0 and in_features % 128 == 0 and rows <= 512:
        if out_features >= 4096:
            if rows <= 128:
                return True
            if rows <= 256:
                if w_bits <= 6:
                    return w_bits <= 5 or out_features <= 16384
                return out_features <= 8192
            return w_bits == 3 and out_features <= 8192
        if out_features >= 1024 and w_bits <= 4:
            return True
    if rows <= min(64, GEMM_MAX_M):
        if in_features > 4096 and ((w_bits >= 6 and out_features >= 5120) or (w_bits >= 5 and out_features <= 2048)):
            return False
        return out_features < 8192 or w_bits <= 5
    return rows <= min(128, GEMM_MAX_M) and 4096 <= out_features < 8192 and 0 < in_features <= 4096


def fused_set_pays(rows: int, out_features, w_bits: int, in_features: int) -> bool:
    """Whether ONE launch of the tiled GEMM over linears that share their input (``gemm_kbit_group``) beats calling them
    one by one, each through whatever ``fused_gemm_pays`` picks (measured on the q/k/v and gate/up sets of the
    Llama-2-7B / Llama-3-8B / 13B layers at 16..256 rows): from 33 rows on -- from 9 where every member has at most
    8192 rows (q/k/v of the 7B layer at 16 rows, 3 bits: 16 us against 23; of the 13B layer: 20 against 36); wide
    members (gate/up) at 9..32 rows are as fast module by module -- up to 128 rows at every bit-width (q/k/v of the 7B layer at 128 rows, 3 bits: 33 us against 44 one by one and
    128 for three dequant + GEMM pairs; gate/up at 8 bits: 96 against 115 for the pairs), up to 256 at up to 6 bits
    (gate/up at 5 bits: 105 against 145) and, at 7 and 8 bits, where every member has fewer than 8192 rows (q/k/v at 8
    bits: 94 against 114; gate/up: 145 against 149); up to 512 at 3 bits where no member has more than 8192 rows, as
    each member alone would."""
    if in_features % 128 or not 8 < rows <= 512 or sum(out_features) < 4096:
        return False
    if rows > 256:      # where every member alone would take the fused GEMM (fused_gemm_pays): 3 bits, up to 8192 rows
        return w_bits == 3 and max(out_features) <= 8192
    if rows <= 32:
        return max(out_features) <= 8192 and in_features >= 1024
    return rows <= 128 or w_bits <= 6 or max(out_features) < 8192


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

"""Tensor-level wrappers of the decode-step kernels (``ap_add_rmsnorm``, ``ap_silu_mul``,
``ap_decode_attention``, ``ap_decode_advance``): argument checks, output allocation, the current stream.

The reference has no counterpart: between its linears it runs the Hugging Face modules
(any_precision/modules/AnyPrecisionForCausalLM.py:88-97).
"""
from __future__ import annotations

import torch

from . import _capi


def _f16(t, name):
    if t.dtype != torch.float16 or not t.is_cuda or not t.is_contiguous():
        raise ValueError(f"{name} must be a contiguous fp16 tensor on the GPU")
    return t


def _stream(t):
    return torch.cuda.current_stream(t.device).cuda_stream


def add_rmsnorm(h, delta, weight, eps, h_out=None, x_out=None):
    """``s = h + delta`` (``delta`` may be None), ``x = rmsnorm(s) * weight`` over the last dimension.
    Returns ``(s, x)``; ``h_out`` may be ``h`` itself."""
    _f16(h, "h"), _f16(weight, "weight")
    if delta is not None and _f16(delta, "delta").shape != h.shape:
        raise ValueError("delta must have the shape of h")
    H = h.shape[-1]
    if weight.shape != (H,):
        raise ValueError("weight must have the length of a row of h")
    h_out = torch.empty_like(h) if h_out is None else _f16(h_out, "h_out")
    x_out = torch.empty_like(h) if x_out is None else _f16(x_out, "x_out")
    if h_out.shape != h.shape or x_out.shape != h.shape:
        raise ValueError("outputs must have the shape of h")
    with torch.cuda.device(h.device):
        _capi.check(_capi.lib.ap_add_rmsnorm(h.data_ptr(), 0 if delta is None else delta.data_ptr(), weight.data_ptr(),
                                             h_out.data_ptr(), x_out.data_ptr(), h.numel() // H, H, float(eps), _stream(h)),
                    "ap_add_rmsnorm")
    return h_out, x_out


def silu_mul(gate, up, out=None):
    """``silu(gate) * up`` elementwise."""
    _f16(gate, "gate"), _f16(up, "up")
    if gate.shape != up.shape:
        raise ValueError("gate and up must have one shape")
    out = torch.empty_like(gate) if out is None else _f16(out, "out")
    if out.shape != gate.shape:
        raise ValueError("out must have the shape of gate")
    with torch.cuda.device(gate.device):
        _capi.check(_capi.lib.ap_silu_mul(gate.data_ptr(), up.data_ptr(), out.data_ptr(), gate.numel(), _stream(gate)),
                    "ap_silu_mul")
    return out


def decode_attention(qkv, cos_table, sin_table, kcache, vcache, pos, n_heads, scale, out=None):
    """Rotary embedding, cache append and attention for one new token.

    ``qkv`` [n_heads + 2 n_kv, hd] (before the rotary embedding); ``cos_table`` / ``sin_table`` fp32
    [max_len, hd / 2]; ``kcache`` / ``vcache`` fp16 [n_kv, max_len, hd], row ``pos`` of each is written;
    ``pos`` an int64 device tensor of one element.  Returns the context [n_heads * hd]."""
    _f16(qkv, "qkv"), _f16(kcache, "kcache"), _f16(vcache, "vcache")
    n_kv, max_len, hd = kcache.shape
    if vcache.shape != kcache.shape or qkv.numel() != (n_heads + 2 * n_kv) * hd:
        raise ValueError("qkv, kcache and vcache do not fit each other")
    for t, name in ((cos_table, "cos_table"), (sin_table, "sin_table")):
        if t.dtype != torch.float32 or not t.is_cuda or not t.is_contiguous() or t.shape != (max_len, hd // 2):
            raise ValueError(f"{name} must be a contiguous fp32 GPU tensor [max_len, head_dim / 2]")
    if pos.dtype != torch.int64 or not pos.is_cuda or pos.numel() != 1:
        raise ValueError("pos must be an int64 GPU tensor of one element")
    out = torch.empty((n_heads * hd,), dtype=torch.float16, device=qkv.device) if out is None else _f16(out, "out")
    if out.numel() != n_heads * hd:
        raise ValueError("out must hold n_heads * head_dim elements")
    with torch.cuda.device(qkv.device):
        _capi.check(_capi.lib.ap_decode_attention(qkv.data_ptr(), cos_table.data_ptr(), sin_table.data_ptr(), kcache.data_ptr(),
                                                  vcache.data_ptr(), pos.data_ptr(), out.data_ptr(), n_heads, n_kv, hd, max_len,
                                                  float(scale), _stream(qkv)), "ap_decode_attention")
    return out


def advance(logits, pos, tok, emitted):
    """The end of a greedy decode step on device scalars: ``t = argmax(logits)`` (first index of the maximum);
    ``pos += 1``; ``emitted[pos] = t`` (if that row exists); ``tok = t``.  ``pos`` and ``tok`` int64 tensors of
    one element, ``emitted`` an int64 vector."""
    _f16(logits, "logits")
    for t, name in ((pos, "pos"), (tok, "tok"), (emitted, "emitted")):
        if t.dtype != torch.int64 or not t.is_cuda or not t.is_contiguous():
            raise ValueError(f"{name} must be a contiguous int64 GPU tensor")
    if pos.numel() != 1 or tok.numel() != 1 or emitted.dim() != 1:
        raise ValueError("pos and tok hold one element each, emitted is a vector")
    with torch.cuda.device(logits.device):
        _capi.check(_capi.lib.ap_decode_advance(logits.data_ptr(), logits.numel(), pos.data_ptr(), tok.data_ptr(),
                                                emitted.data_ptr(), emitted.numel(), _stream(logits)), "ap_decode_advance")

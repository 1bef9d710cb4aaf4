"""Greedy decoding of a Llama-architecture ``AnyPrecisionForCausalLM`` with the decode step
captured in a HIP graph.

The reference times ``model.generate(..., precision=b, max_new_tokens=256)`` through the
Hugging Face loop (demo.py:59-80), which at batch 1 is bound by Python and launch overhead,
not by the kernels.  Here one decode step -- embedding, 32 x (norm, q/k/v GEMV, rotary,
cache write, attention over a static cache, o GEMV, norm, gate/up GEMV, SiLU, down GEMV),
final norm, head, argmax, position increment -- is recorded once per precision and replayed
per token: no host work between tokens.  With ``fused_ops`` (the default) a layer is 7 launches, all
of this library: the seven linears in four (q/k/v as one grouped launch; gate and up as one launch that
also applies SiLU(gate) * up), residual add + RMSNorm twice, rotary + cache append + attention in one kernel.  Without it everything
but the linears is stock PyTorch ops, as in the reference (19 launches per layer); that path also
serves the prompt and is what the fused one is tested against.

Supports Llama-style decoders (RMSNorm, rotary attention with optional grouped KV heads,
SwiGLU MLP, no biases in norms); anything else raises.
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F

from . import _capi
from .decode_ops import advance
from .linear import forward_group, forward_swiglu


def _rope(x, cos, sin_signed):
    """Rotary embedding of x [T, heads, hd] in three kernels: x * cos + rotate_half(x) * sin, with
    rotate_half(x) * sin written as roll(x, hd / 2) * (sin with its first half negated)."""
    return torch.addcmul(torch.roll(x, x.shape[-1] // 2, dims=-1) * sin_signed, x, cos)


class GraphDecoder:
    def __init__(self, ap_model, max_len=512, group_launches=True, fused_ops=True):
        """``group_launches``: issue the q/k/v and the gate/up GEMVs of a layer as one launch each.
        ``fused_ops``: the decode step runs the library's add + RMSNorm, attention and SiLU * up kernels
        instead of stock PyTorch ops (head sizes 32, 64, 128, 256 and caches of up to 8192 rows)."""
        self.group_launches = group_launches
        cfg = ap_model.config
        if getattr(cfg, "model_type", None) != "llama":
            raise NotImplementedError(f"GraphDecoder handles Llama-architecture models, got {cfg.model_type!r}")
        self.ap = ap_model
        self.cfg = cfg
        self.max_len = max_len
        lm = ap_model.model
        self.embed = lm.model.embed_tokens.weight
        self.layers = list(lm.model.layers)
        self.final_norm = lm.model.norm.weight
        self.head = lm.lm_head.weight
        self.eps = cfg.rms_norm_eps
        self.nh = cfg.num_attention_heads
        self.nkv = getattr(cfg, "num_key_value_heads", None) or self.nh
        self.hd = getattr(cfg, "head_dim", None) or cfg.hidden_size // self.nh
        dev = self.embed.device
        if dev.type != "cuda":
            raise RuntimeError("GraphDecoder needs the model on the GPU")
        self.dev = dev
        rope = getattr(cfg, "rope_parameters", None) or {}
        theta = rope.get("rope_theta", None) or getattr(cfg, "rope_theta", 10000.0)
        if rope.get("rope_type", "default") not in ("default", None):
            raise NotImplementedError("only the default rotary embedding is implemented")
        inv = 1.0 / (theta ** (torch.arange(0, self.hd, 2, device=dev, dtype=torch.float32) / self.hd))
        ang = torch.outer(torch.arange(max_len, device=dev, dtype=torch.float32), inv)
        ang = torch.cat((ang, ang), dim=-1)
        self.cos = ang.cos().to(torch.float16)                                              # [max_len, hd]
        sin = ang.sin()
        self.sin_signed = torch.cat((-sin[:, :self.hd // 2], sin[:, self.hd // 2:]), dim=-1).to(torch.float16)
        # additive attention mask, one row per position: 0 up to and including it, -inf beyond
        self.mask = torch.zeros((max_len, max_len), dtype=torch.float16, device=dev)
        self.mask.masked_fill_(torch.arange(max_len, device=dev)[None, :] > torch.arange(max_len, device=dev)[:, None],
                               float("-inf"))
        L = len(self.layers)
        # keys and values of a layer side by side (heads 0..nkv-1 keys, nkv..2nkv-1 values): one write per layer
        self.kvcache = torch.zeros((L, 2 * self.nkv, max_len, self.hd), dtype=torch.float16, device=dev)
        self.kcache = self.kvcache[:, :self.nkv]
        self.vcache = self.kvcache[:, self.nkv:]
        self.head_scale = torch.cat((torch.full((self.nh,), 1.0 / math.sqrt(self.hd)), torch.ones(self.nkv))) \
            .to(torch.float16).to(dev).view(1, self.nh + self.nkv, 1)
        # state the captured step reads and advances
        self.tok = torch.zeros((1,), dtype=torch.long, device=dev)
        self.pos = torch.zeros((1,), dtype=torch.long, device=dev)
        self.emitted = torch.zeros((max_len,), dtype=torch.long, device=dev)
        self.logits = torch.zeros((1, self.head.shape[0]), dtype=torch.float16, device=dev)
        self.graphs = {}
        self.stream = torch.cuda.Stream(device=dev)
        self.fused_ops = bool(fused_ops) and self.hd in (32, 64, 128, 256) and max_len <= 8192
        if self.fused_ops:
            # fp32 rotary tables [max_len, hd / 2] and the static buffers of the fused step
            self.cos32 = ang[:, :self.hd // 2].cos().contiguous()
            self.sin32 = ang[:, :self.hd // 2].sin().contiguous()
            H, I = cfg.hidden_size, cfg.intermediate_size
            f16 = dict(dtype=torch.float16, device=dev)
            self.f_h = torch.zeros((1, H), **f16)        # residual stream
            self.f_x = torch.zeros((1, H), **f16)        # normalised input of the next linears
            self.f_ctx = torch.zeros((1, self.nh * self.hd), **f16)
            self.f_act = torch.zeros((1, I), **f16)

    # ------------------------------------------------------------------ the network
    def _norm(self, x, w):
        return F.rms_norm(x, (x.shape[-1],), w, self.eps)

    def _layer(self, li, h, pos_idx, cos, sin_signed, mask, precision):
        """h [T, H]; pos_idx [T] cache rows of these tokens; mask [nkv, g * T, max_len] additive, fp16.
        Kernel launches per layer and token: 2 norms, 5 for the linears (q/k/v and gate/up grouped),
        3 rotary, 1 cache write, 4 attention (mask copy, scores, softmax, context), 2 residual adds,
        2 for SiLU * up."""
        layer = self.layers[li]
        T = h.shape[0]
        att = layer.self_attn
        nq, nk = self.nh * self.hd, self.nkv * self.hd
        x = self._norm(h, layer.input_layernorm.weight)
        if self.group_launches:
            qkv = forward_group((att.q_proj, att.k_proj, att.v_proj), x, precision, concat=True)       # [T, nq + 2 nk]
        else:
            qkv = torch.cat([m(x, precision=precision) for m in (att.q_proj, att.k_proj, att.v_proj)], dim=-1)
        # rotary over all heads at once: the value heads carry cos = 1, sin = 0; q comes out scaled by 1/sqrt(hd)
        qkv = _rope(qkv.view(T, self.nh + 2 * self.nkv, self.hd), cos, sin_signed)
        self.kvcache[li].index_copy_(1, pos_idx, qkv[:, self.nh:].transpose(0, 1))
        g = self.nh // self.nkv
        qh = qkv[:, :self.nh].transpose(0, 1).reshape(self.nkv, g * T, self.hd)                        # [nkv, g*T, hd]
        scores = torch.baddbmm(mask, qh, self.kcache[li].transpose(1, 2))                              # [nkv, g*T, max_len]
        probs = torch.softmax(scores, dim=-1)
        ctx = torch.bmm(probs, self.vcache[li]).view(self.nh, T, self.hd).transpose(0, 1).reshape(T, nq)
        h = h + att.o_proj(ctx, precision=precision)
        x = self._norm(h, layer.post_attention_layernorm.weight)
        if self.group_launches:
            gate, up = forward_group((layer.mlp.gate_proj, layer.mlp.up_proj), x, precision)
        else:
            gate, up = layer.mlp.gate_proj(x, precision=precision), layer.mlp.up_proj(x, precision=precision)
        return h + layer.mlp.down_proj(F.silu(gate) * up, precision=precision)

    def _forward(self, tokens, pos_idx, precision):
        """tokens [T], pos_idx [T] (device tensors) -> logits of the last token [1, vocab]."""
        T = tokens.shape[0]
        h = self.embed.index_select(0, tokens)
        # per-head rotary factors [T, nh + 2 nkv, hd]: the query heads carry the 1/sqrt(hd) of the attention,
        # the value heads pass through (cos = 1, sin = 0)
        cos = self.cos.index_select(0, pos_idx).unsqueeze(1) * self.head_scale
        sin_signed = self.sin_signed.index_select(0, pos_idx).unsqueeze(1) * self.head_scale
        cos = torch.cat((cos, cos.new_ones((T, self.nkv, self.hd))), dim=1)
        sin_signed = torch.cat((sin_signed, sin_signed.new_zeros((T, self.nkv, self.hd))), dim=1)
        g = self.nh // self.nkv
        mask = self.mask.index_select(0, pos_idx).repeat(g, 1).unsqueeze(0).expand(self.nkv, g * T, self.max_len)
        for li in range(len(self.layers)):
            h = self._layer(li, h, pos_idx, cos, sin_signed, mask, precision)
        h = self._norm(h[-1:], self.final_norm)
        return F.linear(h, self.head)

    def _forward_fused(self, precision):
        """The token self.tok at cache row self.pos through the network -> logits [1, vocab]; 7 launches per layer."""
        lib, st = _capi.lib, torch.cuda.current_stream(self.dev).cuda_stream
        H, eps = self.cfg.hidden_size, float(self.eps)
        scale = 1.0 / math.sqrt(self.hd)

        def add_norm(delta, weight):          # f_h += delta; f_x = rmsnorm(f_h) * weight
            _capi.check(lib.ap_add_rmsnorm(self.f_h.data_ptr(), 0 if delta is None else delta.data_ptr(), weight.data_ptr(),
                                           self.f_h.data_ptr(), self.f_x.data_ptr(), 1, H, eps, st), "ap_add_rmsnorm")

        torch.index_select(self.embed, 0, self.tok, out=self.f_h)
        delta = None
        for li, layer in enumerate(self.layers):
            att = layer.self_attn
            add_norm(delta, layer.input_layernorm.weight)
            if self.group_launches:
                qkv = forward_group((att.q_proj, att.k_proj, att.v_proj), self.f_x, precision, concat=True)
            else:
                qkv = torch.cat([m(self.f_x, precision=precision) for m in (att.q_proj, att.k_proj, att.v_proj)], dim=-1)
            _capi.check(lib.ap_decode_attention(qkv.data_ptr(), self.cos32.data_ptr(), self.sin32.data_ptr(),
                                                self.kcache[li].data_ptr(), self.vcache[li].data_ptr(), self.pos.data_ptr(),
                                                self.f_ctx.data_ptr(), self.nh, self.nkv, self.hd, self.max_len, scale, st),
                        "ap_decode_attention")
            add_norm(att.o_proj(self.f_ctx, precision=precision), layer.post_attention_layernorm.weight)
            if self.group_launches:      # gate, up and the activation function in one launch
                forward_swiglu(layer.mlp.gate_proj, layer.mlp.up_proj, self.f_x, precision, out=self.f_act)
            else:
                gate, up = layer.mlp.gate_proj(self.f_x, precision=precision), layer.mlp.up_proj(self.f_x, precision=precision)
                _capi.check(lib.ap_silu_mul(gate.data_ptr(), up.data_ptr(), self.f_act.data_ptr(), gate.numel(), st), "ap_silu_mul")
            delta = layer.mlp.down_proj(self.f_act, precision=precision)
        add_norm(delta, self.final_norm)
        return torch.mm(self.f_x, self.head.t(), out=self.logits)

    def _step(self, precision):
        """One decode step on the static state: consumes self.tok at self.pos, leaves the next token."""
        if self.fused_ops:
            self._forward_fused(precision)           # writes self.logits
            advance(self.logits, self.pos, self.tok, self.emitted)
            return
        logits = self._forward(self.tok, self.pos, precision)
        self.logits.copy_(logits)
        nxt = torch.argmax(logits, dim=-1)
        self.pos.add_(1)
        self.emitted.index_copy_(0, self.pos, nxt)
        self.tok.copy_(nxt)

    # ------------------------------------------------------------------ driving it
    @torch.inference_mode()
    def prefill(self, input_ids, precision):
        """Runs the prompt [T] through the model (no graph), fills the cache, leaves the first new token."""
        ids = input_ids.reshape(-1).to(self.dev)
        T = ids.numel()
        if T < 1 or T >= self.max_len:
            raise ValueError(f"prompt length {T} outside 1..{self.max_len - 1}")
        self.stream.wait_stream(torch.cuda.current_stream(self.dev))     # the ids may still be in flight there
        with torch.cuda.stream(self.stream):
            self.kvcache.zero_()
            pos_idx = torch.arange(T, device=self.dev)
            logits = self._forward(ids, pos_idx, precision)
            self.logits.copy_(logits)
            nxt = torch.argmax(logits, dim=-1)
            self.emitted.zero_()
            self.emitted[:T] = ids
            self.pos.fill_(T)
            self.emitted.index_copy_(0, self.pos, nxt)
            self.tok.copy_(nxt)
        self.stream.synchronize()

    @torch.inference_mode()
    def capture(self, precision):
        """Records the decode step for ``precision`` (state is saved and restored around the warm-up)."""
        if precision in self.graphs:
            return self.graphs[precision]
        saved = (self.tok.clone(), self.pos.clone(), self.emitted.clone(), self.kvcache.clone())
        with torch.cuda.stream(self.stream):
            self.pos.clamp_(max=self.max_len - 4)
            for _ in range(2):
                self._step(precision)            # warm-up: library handles, allocator pools
            self.stream.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=self.stream):
                self._step(precision)
        self.stream.synchronize()
        for dst, src in zip((self.tok, self.pos, self.emitted, self.kvcache), saved):
            dst.copy_(src)
        torch.cuda.synchronize()
        self.graphs[precision] = g
        return g

    @torch.inference_mode()
    def decode(self, steps, precision, use_graph=True):
        """``steps`` further tokens after a prefill; returns all token ids so far [pos + 1]."""
        start = int(self.pos.item())
        if start + steps >= self.max_len:
            raise ValueError(f"{start} + {steps} tokens do not fit the cache of {self.max_len}")
        if use_graph:
            g = self.capture(precision)
            with torch.cuda.stream(self.stream):
                for _ in range(steps):
                    g.replay()
        else:
            with torch.cuda.stream(self.stream):
                for _ in range(steps):
                    self._step(precision)
        self.stream.synchronize()
        return self.emitted[:start + steps + 1].clone()

    @torch.inference_mode()
    def generate(self, input_ids, max_new_tokens, precision=None, use_graph=True):
        """Greedy continuation of ``input_ids`` [T] by ``max_new_tokens`` tokens -> ids [T + max_new_tokens]."""
        precision = self.ap.precision if precision is None else precision
        if precision not in self.ap.precisions:
            raise RuntimeError(f"{self.ap.precisions}-bit precisions are supported but {precision}-bit was specified.")
        self.prefill(input_ids, precision)
        if max_new_tokens > 1:
            return self.decode(max_new_tokens - 1, precision, use_graph)
        return self.emitted[:int(self.pos.item()) + 1].clone()

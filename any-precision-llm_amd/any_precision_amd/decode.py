"""Greedy decoding of a Llama-architecture ``AnyPrecisionForCausalLM`` with the decode step
captured in a HIP graph.

The reference times ``model.generate(..., precision=b, max_new_tokens=256)`` through the
Hugging Face loop (demo.py:59-80), which at batch 1 is bound by Python and launch overhead,
not by the kernels.  Here one decode step -- embedding, 32 x (norm, q/k/v GEMV, rotary,
cache write, attention over a static cache, o GEMV, norm, gate/up GEMV, SiLU, down GEMV),
final norm, head, argmax, position increment -- is recorded once per precision and replayed
per token: no host work between tokens.  Only the seven linears per layer are this
library's kernels (q/k/v and gate/up as one grouped launch each); everything else is stock
PyTorch ops, as in the reference.

Supports Llama-style decoders (RMSNorm, rotary attention with optional grouped KV heads,
SwiGLU MLP, no biases in norms); anything else raises.
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F

from .linear import forward_group


def _rotate_half(x):
    h = x.shape[-1] // 2
    return torch.cat((-x[..., h:], x[..., :h]), dim=-1)


class GraphDecoder:
    def __init__(self, ap_model, max_len=512, group_launches=True):
        """``group_launches``: issue the q/k/v and the gate/up GEMVs of a layer as one launch each."""
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
        self.cos, self.sin = ang.cos().to(torch.float16), ang.sin().to(torch.float16)     # [max_len, hd]
        L = len(self.layers)
        self.kcache = torch.zeros((L, self.nkv, max_len, self.hd), dtype=torch.float16, device=dev)
        self.vcache = torch.zeros_like(self.kcache)
        self.arange = torch.arange(max_len, device=dev)
        # state the captured step reads and advances
        self.tok = torch.zeros((1,), dtype=torch.long, device=dev)
        self.pos = torch.zeros((1,), dtype=torch.long, device=dev)
        self.emitted = torch.zeros((max_len,), dtype=torch.long, device=dev)
        self.logits = torch.zeros((1, self.head.shape[0]), dtype=torch.float16, device=dev)
        self.graphs = {}
        self.stream = torch.cuda.Stream(device=dev)

    # ------------------------------------------------------------------ the network
    def _group(self, modules, x, precision):
        if self.group_launches:
            return forward_group(modules, x, precision)
        return [m(x, precision=precision) for m in modules]

    def _norm(self, x, w):
        return F.rms_norm(x, (x.shape[-1],), w, self.eps)

    def _layer(self, li, h, pos_idx, cos, sin, mask, precision):
        """h [T, H]; pos_idx [T] cache rows of these tokens; mask [T, max_len] additive."""
        layer = self.layers[li]
        T = h.shape[0]
        x = self._norm(h, layer.input_layernorm.weight)
        att_in = layer.self_attn
        q, k, v = self._group((att_in.q_proj, att_in.k_proj, att_in.v_proj), x, precision)
        q, k, v = q.view(T, self.nh, self.hd), k.view(T, self.nkv, self.hd), v.view(T, self.nkv, self.hd)
        q = q * cos + _rotate_half(q) * sin
        k = k * cos + _rotate_half(k) * sin
        self.kcache[li].index_copy_(1, pos_idx, k.transpose(0, 1))
        self.vcache[li].index_copy_(1, pos_idx, v.transpose(0, 1))
        g = self.nh // self.nkv
        qh = q.transpose(0, 1).reshape(self.nkv, g * T, self.hd)                        # [nkv, g*T, hd]
        scores = torch.bmm(qh, self.kcache[li].transpose(1, 2)).float() / math.sqrt(self.hd)   # [nkv, g*T, max_len]
        scores = scores.view(self.nkv, g, T, self.max_len) + mask
        probs = torch.softmax(scores, dim=-1).to(torch.float16).view(self.nkv, g * T, self.max_len)
        att = torch.bmm(probs, self.vcache[li]).view(self.nh, T, self.hd).transpose(0, 1).reshape(T, self.nh * self.hd)
        h = h + layer.self_attn.o_proj(att, precision=precision)
        x = self._norm(h, layer.post_attention_layernorm.weight)
        gate, up = self._group((layer.mlp.gate_proj, layer.mlp.up_proj), x, precision)
        return h + layer.mlp.down_proj(F.silu(gate) * up, precision=precision)

    def _forward(self, tokens, pos_idx, precision):
        """tokens [T], pos_idx [T] (device tensors) -> logits of the last token [1, vocab]."""
        h = self.embed.index_select(0, tokens)
        cos = self.cos.index_select(0, pos_idx).unsqueeze(1)
        sin = self.sin.index_select(0, pos_idx).unsqueeze(1)
        mask = torch.where(self.arange.unsqueeze(0) > pos_idx.unsqueeze(1), float("-inf"), 0.0)   # [T, max_len] fp32
        for li in range(len(self.layers)):
            h = self._layer(li, h, pos_idx, cos, sin, mask, precision)
        h = self._norm(h[-1:], self.final_norm)
        return F.linear(h, self.head)

    def _step(self, precision):
        """One decode step on the static state: consumes self.tok at self.pos, leaves the next token."""
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
            self.kcache.zero_()
            self.vcache.zero_()
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
        saved = (self.tok.clone(), self.pos.clone(), self.emitted.clone(), self.kcache.clone(), self.vcache.clone())
        with torch.cuda.stream(self.stream):
            self.pos.clamp_(max=self.max_len - 4)
            for _ in range(2):
                self._step(precision)            # warm-up: library handles, allocator pools
            self.stream.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=self.stream):
                self._step(precision)
        self.stream.synchronize()
        for dst, src in zip((self.tok, self.pos, self.emitted, self.kcache, self.vcache), saved):
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

"""Decode-step kernels (add + RMSNorm, SiLU * up, rotary + cache append + attention) against plain
PyTorch fp32 statements of the same operators, through the C ABI.

Tolerances (fp16 outputs of fp32 arithmetic, one rounding): 2e-3 relative to the largest reference
magnitude for the element-wise kernels, 4e-3 for attention (its inputs are rounded cache rows)."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu


def _close(got, want, tol, what):
    got, want = got.float(), want.float()
    assert torch.isfinite(got).all(), what
    err = (got - want).abs().max().item()
    assert err <= tol * max(want.abs().max().item(), 1e-6), f"{what}: max abs err {err:.3e}, max |ref| {want.abs().max().item():.3e}"


@pytest.mark.parametrize("rows,H", [(1, 128), (1, 4096), (3, 11008), (2, 8), (1, 5120)])
def test_add_rmsnorm_matches_fp32(rows, H):
    from any_precision_amd.decode_ops import add_rmsnorm
    g = torch.Generator(device="cuda").manual_seed(rows * 100003 + H)
    h = torch.randn((rows, H), device="cuda", generator=g).half()
    d = (torch.randn((rows, H), device="cuda", generator=g) * 0.5).half()
    w = (1 + 0.1 * torch.randn((H,), device="cuda", generator=g)).half()
    for delta in (None, d):
        print(f"add_rmsnorm rows={rows} H={H} delta={delta is not None}", flush=True)
        s, x = add_rmsnorm(h, delta, w, 1e-5)
        want_s = h if delta is None else (h.float() + d.float()).half()
        assert torch.equal(s, want_s)                                   # the residual stream is an fp16 add: exact
        f = want_s.float()
        want_x = f * torch.rsqrt(f.pow(2).mean(-1, keepdim=True) + 1e-5) * w.float()
        _close(x, want_x, 2e-3, f"rmsnorm rows={rows} H={H}")
    # in place on the residual stream
    h2 = h.clone()
    s, x = add_rmsnorm(h2, d, w, 1e-5, h_out=h2)
    assert s.data_ptr() == h2.data_ptr() and torch.equal(h2, (h.float() + d.float()).half())


@pytest.mark.parametrize("n", [8, 352, 11008, 14336 * 3])
def test_silu_mul_matches_fp32(n):
    from any_precision_amd.decode_ops import silu_mul
    g = torch.Generator(device="cuda").manual_seed(n)
    gate = (torch.randn((n,), device="cuda", generator=g) * 3).half()
    up = torch.randn((n,), device="cuda", generator=g).half()
    print(f"silu_mul n={n}", flush=True)
    got = silu_mul(gate, up)
    want = torch.nn.functional.silu(gate.float()) * up.float()
    _close(got, want, 2e-3, f"silu_mul n={n}")


def _rotary_tables(max_len, hd, theta=10000.0):
    inv = 1.0 / (theta ** (torch.arange(0, hd, 2, device="cuda", dtype=torch.float32) / hd))
    ang = torch.outer(torch.arange(max_len, device="cuda", dtype=torch.float32), inv)
    return ang.cos().contiguous(), ang.sin().contiguous()


def _attention_reference(qkv, cos, sin, kcache, vcache, pos, nh, scale):
    """fp32 statement: rotate q and k (x * cos + rotate_half(x) * sin), append k (rounded to fp16) and v at row pos,
    softmax(scale * q k^T) v over rows 0..pos with query head h on key/value head h // (nh // nkv)."""
    nkv, max_len, hd = kcache.shape
    x = qkv.float().view(nh + 2 * nkv, hd)
    c, s = torch.cat((cos[pos], cos[pos])), torch.cat((sin[pos], sin[pos]))
    rot = lambda t: t * c + torch.cat((-t[:, hd // 2:], t[:, :hd // 2]), dim=1) * s
    q, k, v = rot(x[:nh]), rot(x[nh:nh + nkv]).half(), x[nh + nkv:].half()
    K = torch.cat((kcache[:, :pos].float(), k.float().unsqueeze(1)), dim=1)       # [nkv, pos + 1, hd]
    V = torch.cat((vcache[:, :pos].float(), v.float().unsqueeze(1)), dim=1)
    g = nh // nkv
    out = torch.empty((nh, hd), device="cuda")
    for h in range(nh):
        p = torch.softmax(scale * (K[h // g] @ q[h]), dim=0)
        out[h] = p @ V[h // g]
    return out.reshape(-1), k, v


@pytest.mark.parametrize("nh,nkv,hd", [(4, 2, 32), (8, 8, 64), (32, 32, 128), (8, 1, 128), (4, 2, 256)])
def test_decode_attention_matches_fp32(nh, nkv, hd):
    from any_precision_amd.decode_ops import decode_attention
    max_len = 400
    cos, sin = _rotary_tables(max_len, hd)
    g = torch.Generator(device="cuda").manual_seed(nh * 1000 + hd)
    scale = 1.0 / math.sqrt(hd)
    for pos in (0, 1, 63, 64, 65, 257, max_len - 1):
        print(f"decode_attention nh={nh} nkv={nkv} hd={hd} pos={pos}", flush=True)
        kcache = torch.randn((nkv, max_len, hd), device="cuda", generator=g).half()
        vcache = torch.randn((nkv, max_len, hd), device="cuda", generator=g).half()
        qkv = torch.randn((nh + 2 * nkv, hd), device="cuda", generator=g).half()
        k0, v0 = kcache.clone(), vcache.clone()
        p = torch.tensor([pos], dtype=torch.int64, device="cuda")
        want, k_new, v_new = _attention_reference(qkv, cos, sin, k0, v0, pos, nh, scale)
        got = decode_attention(qkv, cos, sin, kcache, vcache, p, nh, scale)
        _close(got, want, 4e-3, f"context pos={pos}")
        # the cache: row pos holds the rotated key (within an fp16 ulp of the fp32 statement) and the value; no other row changed
        _close(kcache[:, pos], k_new, 2e-3, f"key row pos={pos}")
        assert torch.equal(vcache[:, pos], v_new)
        keep = torch.ones(max_len, dtype=torch.bool, device="cuda")
        keep[pos] = False
        assert torch.equal(kcache[:, keep], k0[:, keep]) and torch.equal(vcache[:, keep], v0[:, keep])


def test_decode_attention_ignores_a_position_outside_the_cache():
    from any_precision_amd.decode_ops import decode_attention
    nh, nkv, hd, max_len = 4, 2, 64, 48
    cos, sin = _rotary_tables(max_len, hd)
    g = torch.Generator(device="cuda").manual_seed(7)
    kcache = torch.randn((nkv, max_len, hd), device="cuda", generator=g).half()
    vcache = torch.randn((nkv, max_len, hd), device="cuda", generator=g).half()
    qkv = torch.randn((nh + 2 * nkv, hd), device="cuda", generator=g).half()
    k0, v0 = kcache.clone(), vcache.clone()
    out = torch.full((nh * hd,), 7.0, dtype=torch.float16, device="cuda")
    for bad in (max_len, -1, 1 << 40):
        p = torch.tensor([bad], dtype=torch.int64, device="cuda")
        decode_attention(qkv, cos, sin, kcache, vcache, p, nh, 0.125, out=out)
        torch.cuda.synchronize()
        assert torch.equal(kcache, k0) and torch.equal(vcache, v0) and bool((out == 7.0).all())


def test_fused_step_follows_the_stock_step(tmp_path):
    """The decoder with the library's step kernels against the same decoder on stock PyTorch ops: same
    prompt, logits of every step within 2e-2 of the largest logit, equal tokens wherever the stock step's
    top-2 margin exceeds that; graph replay equals the eager fused step bit for bit."""
    from test_model_checkpoint import tiny_config
    from any_precision_amd import AnyPrecisionForCausalLM, GraphDecoder
    ap = AnyPrecisionForCausalLM.from_config(tiny_config(), seed=5, device="cuda")
    fused = GraphDecoder(ap, max_len=64)
    stock = GraphDecoder(ap, max_len=64, fused_ops=False)
    assert fused.fused_ops and not stock.fused_ops
    ids = torch.randint(0, 320, (9,), generator=torch.Generator().manual_seed(1)).cuda()
    for b in (3, 8):
        print(f"fused step b={b}", flush=True)
        with_graph = fused.generate(ids, 12, precision=b, use_graph=True)
        eager = fused.generate(ids, 12, precision=b, use_graph=False)
        assert torch.equal(with_graph, eager)
        # step by step on the stock decoder's own token sequence
        stock.prefill(ids, b)
        fused.prefill(ids, b)
        for step in range(10):
            assert torch.equal(stock.tok, fused.tok), f"step {step}"
            stock.decode(1, b, use_graph=False)
            fused.decode(1, b, use_graph=False)
            want, got = stock.logits[0].float(), fused.logits[0].float()
            tol = 2e-2 * want.abs().max().item()
            assert (got - want).abs().max().item() <= tol, f"step {step}"
            top2 = want.topk(2).values
            if (top2[0] - top2[1]).item() <= 2 * tol:
                fused.tok.copy_(stock.tok)               # a near tie: keep both on the stock sequence
                fused.emitted.copy_(stock.emitted)


def test_fused_step_at_llama3_8b_width_with_grouped_kv_heads():
    """Two decoder layers at Llama-3-8B width (hidden 4096, FFN 14336, 32 query heads on 8 key/value heads of 128):
    the one-launch q/k/v, attention, SwiGLU and add + norm kernels at their real shapes.  Graph replay equals the
    eager fused step; against the stock-ops step the logits agree within 2e-2 of the largest and the greedy tokens
    are equal wherever the stock step's top-2 margin exceeds twice that."""
    from transformers import LlamaConfig
    from any_precision_amd import AnyPrecisionForCausalLM, GraphDecoder
    cfg = LlamaConfig(hidden_size=4096, intermediate_size=14336, num_hidden_layers=2, num_attention_heads=32,
                      num_key_value_heads=8, vocab_size=32000, max_position_embeddings=8192, rms_norm_eps=1e-5,
                      rope_theta=500000.0, tie_word_embeddings=False)
    ap = AnyPrecisionForCausalLM.from_config(cfg, seed=2, device="cuda")
    fused, stock = GraphDecoder(ap, max_len=128), GraphDecoder(ap, max_len=128, fused_ops=False)
    ids = torch.randint(0, 32000, (70,), generator=torch.Generator().manual_seed(3)).cuda()
    for b in (3, 8):
        print(f"llama-3 width b={b}", flush=True)
        assert torch.equal(fused.generate(ids, 10, precision=b, use_graph=True), fused.generate(ids, 10, precision=b, use_graph=False))
        stock.prefill(ids, b)
        fused.prefill(ids, b)
        for step in range(6):
            assert torch.equal(stock.tok, fused.tok), f"b={b} step {step}"
            stock.decode(1, b, use_graph=False)
            fused.decode(1, b, use_graph=False)
            want, got = stock.logits[0].float(), fused.logits[0].float()
            tol = 2e-2 * want.abs().max().item()
            assert (got - want).abs().max().item() <= tol, f"b={b} step {step}"
            top2 = want.topk(2).values
            if (top2[0] - top2[1]).item() <= 2 * tol:
                fused.tok.copy_(stock.tok)
                fused.emitted.copy_(stock.emitted)


@pytest.mark.parametrize("n", [1, 7, 8, 320, 32000, 128256 + 3])
def test_advance_is_argmax_and_bookkeeping(n):
    """ap_decode_advance against torch.argmax (first index of the maximum, NaN as the maximum) and the three
    scalar updates it replaces; a position at the end of the buffer moves nothing but the token."""
    from any_precision_amd.decode_ops import advance
    g = torch.Generator(device="cuda").manual_seed(n)
    for case in ("random", "ties", "nan", "neg_inf"):
        logits = torch.randn((1, n), device="cuda", generator=g).half()
        if case == "ties":
            logits = (logits * 2).round() / 2                      # many equal maxima
        elif case == "nan" and n > 2:
            logits[0, n // 2] = float("nan")
            logits[0, n - 1] = float("nan")
        elif case == "neg_inf":
            logits.fill_(float("-inf"))
        print(f"advance n={n} {case}", flush=True)
        want = int(torch.argmax(logits, dim=-1).item())
        pos = torch.tensor([5], device="cuda")
        tok = torch.tensor([-1], device="cuda")
        emitted = torch.full((16,), -7, device="cuda")
        advance(logits, pos, tok, emitted)
        assert int(tok.item()) == want and int(pos.item()) == 6 and int(emitted[6].item()) == want
        assert (emitted[:6] == -7).all() and (emitted[7:] == -7).all()
        pos.fill_(15)                                              # no row 16: only the token changes
        tok.fill_(-1)
        advance(logits, pos, tok, emitted)
        assert int(tok.item()) == want and int(pos.item()) == 15 and int(emitted[15].item()) == -7

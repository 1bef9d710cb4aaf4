"""AnyPrecisionForCausalLM and GraphDecoder on the GPU against a plain fp16 Hugging Face model
that holds the dequantised weights (the dense reconstruction of the same precision).

Tolerance: both sides compute in fp16 with fp32 accumulation but in different orders, so
logits are compared at 2e-2 of the largest logit magnitude (two decoder layers)."""
import pytest
import torch

from test_model_checkpoint import tiny_config

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def pair():
    from transformers import LlamaForCausalLM
    from any_precision_amd import AnyPrecisionForCausalLM
    ap = AnyPrecisionForCausalLM.from_config(tiny_config(), seed=5, device="cuda")
    dense = {}
    for b in (3, 8):
        m = LlamaForCausalLM(tiny_config()).half().cuda().eval()
        missing, unexpected = m.load_state_dict(ap.dense_state_dict(b), strict=False)
        assert not unexpected and all("rotary" in k for k in missing), (missing, unexpected)
        dense[b] = m
    return ap, dense


def _close(a, b, what):
    a, b = a.float(), b.float()
    assert torch.isfinite(a).all(), what
    err = (a - b).abs().max().item()
    assert err <= 2e-2 * b.abs().max().item(), f"{what}: max abs err {err:.3e} vs max |ref| {b.abs().max().item():.3e}"


def test_dense_reconstruction_is_the_table_lookup(pair):
    ap, dense = pair
    lin = ap.ap_linears[0]
    from any_precision_amd.packing import unpack_codes
    codes = torch.from_numpy(unpack_codes(lin.qweight.cpu().numpy(), 3).astype("int64")).cuda()
    want = torch.gather(lin.lut3, 1, codes)
    got = dense[3].model.layers[0].self_attn.q_proj.weight
    assert torch.equal(got, want)


@pytest.mark.parametrize("T", [1, 5, 12, 40])     # GEMV kernel, MFMA kernel, fused GEMM, dequant + matmul
def test_forward_matches_the_dense_model(pair, T):
    ap, dense = pair
    ids = torch.randint(0, 320, (1, T), generator=torch.Generator().manual_seed(T)).cuda()
    for b in (3, 8):
        print(f"model forward T={T} b={b}", flush=True)
        with torch.inference_mode():
            got = ap(ids, precision=b).logits
            want = dense[b](ids).logits
        assert got.shape == (1, T, 320)
        _close(got, want, f"T={T} b={b}")
    assert ap.precision == 8       # restored after the call


def test_generate_switches_precision_and_restores_it(pair):
    ap, dense = pair
    ids = torch.randint(0, 320, (1, 6), generator=torch.Generator().manual_seed(0)).cuda()
    out = ap.generate(ids, precision=3, max_new_tokens=4, do_sample=False, pad_token_id=0)
    assert out.shape == (1, 10) and torch.equal(out[:, :6], ids) and ap.precision == 8


def test_graph_decoder_matches_eager_and_the_dense_model(pair):
    from any_precision_amd import GraphDecoder
    ap, dense = pair
    dec = GraphDecoder(ap, max_len=64)
    ids = torch.randint(0, 320, (9,), generator=torch.Generator().manual_seed(1)).cuda()
    for b in (3, 8):
        print(f"graph decoder b={b}", flush=True)
        with_graph = dec.generate(ids, 12, precision=b, use_graph=True)
        eager = dec.generate(ids, 12, precision=b, use_graph=False)
        again = dec.generate(ids, 12, precision=b, use_graph=True)     # replays after eager work in between
        assert with_graph.shape == (21,) and torch.equal(with_graph[:9], ids)
        assert torch.equal(with_graph, eager) and torch.equal(with_graph, again)
        ungrouped = GraphDecoder(ap, max_len=64, group_launches=False).generate(ids, 12, precision=b)
        assert torch.equal(with_graph, ungrouped)       # grouped launches give the same bits
        # the logits that chose the last token, against the dense model on the same prefix
        with torch.inference_mode():
            want = dense[b](with_graph[:-1].unsqueeze(0)).logits[0, -1]
        _close(dec.logits[0], want, f"decoder logits b={b}")
        # greedy choice agrees wherever the dense model's top-2 margin exceeds the tolerance
        top2 = want.float().topk(2).values
        if (top2[0] - top2[1]).item() > 4e-2 * want.abs().max().item():
            assert int(with_graph[-1]) == int(want.argmax())


def test_opt_layout_with_biased_linears():
    """A second module layout (the reference's analyzer/architectures/opt.yaml: model.decoder.layers,
    q/k/v/out_proj, fc1, fc2) whose linears carry biases (AnyPrecisionLinear.py:40-46,68-69), through
    from_config -> save_quantized -> from_quantized, against the dense model of the same weights."""
    import tempfile
    from transformers import OPTConfig, OPTForCausalLM
    from any_precision_amd import AnyPrecisionForCausalLM

    def config():
        cfg = OPTConfig(hidden_size=64, ffn_dim=160, num_hidden_layers=2, num_attention_heads=4, vocab_size=320,
                        max_position_embeddings=64, word_embed_proj_dim=64, do_layer_norm_before=True)
        cfg.anyprec = {"seed_precision": 3, "parent_precision": 8, "group_count": 1,
                       "arch_config": {"model_name": "model.decoder", "layers_name": "layers",
                                       "module_names": ["self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj",
                                                        "self_attn.out_proj", "fc1", "fc2"]}}
        return cfg

    ap = AnyPrecisionForCausalLM.from_config(config(), seed=2, device="cuda")
    assert len(ap.ap_linears) == 12 and all(m.bias is not None for m in ap.ap_linears)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(3)
    for m in ap.ap_linears:                     # non-trivial biases
        m.bias.copy_(torch.randn(m.bias.shape, device="cuda", generator=gen) * 0.05)
    with tempfile.TemporaryDirectory() as d:
        ap.save_quantized(d)
        back = AnyPrecisionForCausalLM.from_quantized(d).cuda()
    ids = torch.randint(0, 320, (1, 7), generator=torch.Generator().manual_seed(0)).cuda()
    for b in (3, 8):
        dense = OPTForCausalLM(config()).half().cuda().eval()
        missing, unexpected = dense.load_state_dict(ap.dense_state_dict(b), strict=False)
        assert not unexpected and not missing, (missing, unexpected)
        with torch.inference_mode():
            want = dense(ids).logits
            got = ap(ids, precision=b).logits
            got_back = back(ids, precision=b).logits
        _close(got, want, f"opt b={b}")
        assert torch.equal(got, got_back), "model reloaded from its checkpoint differs"

"""The random-init Llama-2-7B-shaped model at its real size (32 layers, hidden 4096, FFN 11008, 32 heads,
vocab 32000; every linear as 8-bit-parent bitplanes, about 8 GB on the GPU): a 128-token prompt, then
tokens decoded from the HIP graph and eagerly, at 3 and 8 bits -- the loop the reference's demo times
(demo.py:59-80) -- and the linears of layer 0 against the oracle on that layer's own buffers."""
import numpy as np
import pytest
import torch

from _util import assert_close_gemv

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def model():
    from transformers import LlamaConfig
    from any_precision_amd import AnyPrecisionForCausalLM
    cfg = LlamaConfig(hidden_size=4096, intermediate_size=11008, num_hidden_layers=32, num_attention_heads=32,
                      num_key_value_heads=32, vocab_size=32000, max_position_embeddings=4096, rms_norm_eps=1e-5,
                      tie_word_embeddings=False)
    print("building the 32-layer model", flush=True)
    m = AnyPrecisionForCausalLM.from_config(cfg, seed=0, device="cuda")
    assert len(m.ap_linears) == 7 * 32
    return m


def test_graph_decode_equals_eager_decode_after_a_128_token_prompt(model):
    from any_precision_amd import GraphDecoder
    dec = GraphDecoder(model, max_len=160)
    ids = torch.randint(0, 32000, (128,), generator=torch.Generator().manual_seed(0)).cuda()
    for b in (3, 8):
        print(f"7B-shaped model: prompt 128 + 8 tokens, w_bits {b}", flush=True)
        with_graph = dec.generate(ids, 9, precision=b, use_graph=True)
        eager = dec.generate(ids, 9, precision=b, use_graph=False)
        assert with_graph.shape == (137,) and torch.equal(with_graph[:128], ids)
        assert torch.equal(with_graph, eager), (with_graph[128:], eager[128:])
        assert torch.isfinite(dec.logits).all()
        assert int(with_graph[128:].min()) >= 0 and int(with_graph[128:].max()) < 32000
    assert model.precision == 8


def test_layer0_linears_match_the_oracle_on_their_own_buffers(model, oracle):
    """q_proj (4096 x 4096) and down_proj (4096 x 11008) of layer 0 through the module's forward -- batch 1
    (GEMV), 4 (matrix-core GEMV) and 16 rows (fused GEMM) -- against the oracle fed the same planes and
    tables copied back from the GPU."""
    layer = model.get_model_layers()[0]
    for name, lin in (("q_proj", layer.self_attn.q_proj), ("down_proj", layer.mlp.down_proj)):
        qw = lin.qweight.cpu().numpy()
        K = lin.in_features
        for b in (3, 8):
            lut = lin._buffers[f"lut{b}"].cpu().numpy()
            for M in (1, 4, 16):
                print(f"layer 0 {name} w_bits {b} M={M}", flush=True)
                x = np.random.default_rng(M).normal(0, 1, size=(M, K)).astype(np.float16)
                with torch.inference_mode():
                    got = lin(torch.from_numpy(x).cuda(), precision=b)
                _, want = oracle.matmul_kbit(x, qw, lut, b, return_f64=True)
                assert_close_gemv(got, want, f"{name} b={b} M={M}")

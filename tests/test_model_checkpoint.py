"""AnyPrecisionForCausalLM on the CPU: module swap, state-dict naming as the reference packer
writes it (pack.py:101-112,165-177), checkpoint directory round trip, precision bookkeeping.
No kernel runs here."""
import json
import os

import pytest
import torch


def tiny_config():
    from transformers import LlamaConfig
    return LlamaConfig(hidden_size=128, intermediate_size=352, num_hidden_layers=2, num_attention_heads=4,
                       num_key_value_heads=2, vocab_size=320, max_position_embeddings=128, rms_norm_eps=1e-5,
                       tie_word_embeddings=False)


@pytest.fixture(scope="module")
def model():
    from any_precision_amd import AnyPrecisionForCausalLM
    return AnyPrecisionForCausalLM.from_config(tiny_config(), seed=3, device="cpu")


def test_linears_are_swapped_and_named_like_the_reference(model):
    from any_precision_amd import AnyPrecisionLinear
    assert len(model.ap_linears) == 2 * 7 and all(isinstance(m, AnyPrecisionLinear) for m in model.ap_linears)
    sd = model.model.state_dict()
    for li in range(2):
        for name, N, K in (("self_attn.q_proj", 128, 128), ("self_attn.k_proj", 64, 128), ("mlp.gate_proj", 352, 128),
                           ("mlp.down_proj", 128, 352)):
            q = sd[f"model.layers.{li}.{name}.qweight"]
            assert q.shape == (8, N, K // 32) and q.dtype == torch.int32
            for b in range(3, 9):
                t = sd[f"model.layers.{li}.{name}.lut{b}"]
                assert t.shape == (N, 1 << b) and t.dtype == torch.float16
            assert f"model.layers.{li}.{name}.weight" not in sd
    assert sd["model.embed_tokens.weight"].shape == (320, 128) and sd["lm_head.weight"].dtype == torch.float16
    assert model.layer_type == "LlamaDecoderLayer" and len(model.get_model_layers()) == 2
    assert model.supported_bits == [3, 4, 5, 6, 7, 8] and model.precision == 8


def test_set_precision_reaches_every_linear(model):
    model.set_precision(4)
    assert model.precision == 4 and all(m.precision == 4 for m in model.ap_linears)
    with pytest.raises(RuntimeError):
        model.set_precision(2)
    model.set_precision(8)


def test_checkpoint_directory_round_trip(model, tmp_path):
    from any_precision_amd import AnyPrecisionForCausalLM
    model.save_quantized(str(tmp_path))
    cfg = json.load(open(os.path.join(tmp_path, "config.json")))
    assert cfg["anyprec"]["seed_precision"] == 3 and cfg["anyprec"]["parent_precision"] == 8
    assert cfg["anyprec"]["arch_config"]["module_names"][0] == "self_attn.q_proj"
    # the file holds plain tensors only: the safe loader reads it
    raw = torch.load(os.path.join(tmp_path, "pytorch_model.bin"), weights_only=True)
    assert raw["model.layers.1.mlp.up_proj.qweight"].dtype == torch.int32

    again = AnyPrecisionForCausalLM.from_quantized(str(tmp_path))
    a, b = model.model.state_dict(), again.model.state_dict()
    assert sorted(a) == sorted(b)
    for k in a:
        assert torch.equal(a[k], b[k]), k

    pruned = AnyPrecisionForCausalLM.from_quantized(str(tmp_path), precisions=[3, 5])
    assert pruned.precision == 5
    lin = pruned.ap_linears[0]
    assert lin.qweight.shape[0] == 5 and hasattr(lin, "lut3") and not hasattr(lin, "lut8")
    assert torch.equal(lin.qweight, model.ap_linears[0].qweight[:5])
    # a model that holds a subset of the precisions has dropped planes and tables the config still promises:
    # saving it would write a checkpoint that cannot be loaded again
    with pytest.raises(RuntimeError, match="every precision"):
        pruned.save_quantized(str(tmp_path / "pruned"))
    assert not os.path.exists(tmp_path / "pruned")


def test_rejects_foreign_checkpoints(tmp_path):
    from any_precision_amd import AnyPrecisionForCausalLM
    cfg = tiny_config()
    with pytest.raises(ValueError):
        AnyPrecisionForCausalLM(None, cfg)
    cfg.anyprec = {"seed_precision": 3, "parent_precision": 8, "group_count": 2, "arch_config": {}}
    with pytest.raises(ValueError):
        AnyPrecisionForCausalLM(None, cfg)

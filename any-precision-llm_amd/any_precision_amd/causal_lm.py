"""``AnyPrecisionForCausalLM``: counterpart of the reference model wrapper
(any_precision/modules/AnyPrecisionForCausalLM.py:29-174) on top of the HIP ops.

Same surface: ``from_quantized(path, precisions=None)``, ``forward(..., precision=b)``,
``generate(..., precision=b)``, ``set_precision``, ``prune_precisions``,
``get_model_layers``, ``layer_type``, ``device``.  The checkpoint directory is the one the
reference packer writes (pack.py:165-177): ``config.json`` with an ``anyprec`` entry
(``seed_precision``, ``parent_precision``, ``group_count``, ``arch_config``) and a
``pytorch_model.bin`` whose linears are stored as ``<module>.qweight`` / ``<module>.lut{b}``
(pack.py:101-112).  The file is read with ``torch.load(weights_only=True)``: nothing in it is
executed.

Beyond the reference: ``from_config`` builds a randomly initialised model of a given shape
(benchmarks, tests), ``save_quantized`` writes the checkpoint directory, ``dense_state_dict``
rebuilds the fp16 weights of one precision (the reference does that on the CPU, one table
lookup per group, evaluate/eval.py:97-110; here it is one ``dequant_kbit`` per linear).
"""
from __future__ import annotations

import gc
import os

import torch
import torch.nn as nn

from .linear import AnyPrecisionLinear

# module layout of the architectures the reference describes (analyzer/architectures/*.yaml)
LLAMA_ARCH_CONFIG = {
    "model_name": "model",
    "layers_name": "layers",
    "module_names": ["self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj", "self_attn.o_proj",
                     "mlp.gate_proj", "mlp.up_proj", "mlp.down_proj"],
}


def _get_by_name(root, dotted):
    """Sub-module ``a.b.0.c`` of ``root`` (numeric parts index into module lists)."""
    for part in dotted.split("."):
        root = root[int(part)] if part.isdigit() else getattr(root, part)
    return root


def _set_by_name(root, dotted, module):
    """Puts ``module`` where ``dotted`` names a sub-module of ``root``."""
    parent, _, leaf = dotted.rpartition(".")
    setattr(_get_by_name(root, parent) if parent else root, leaf, module)


class AnyPrecisionForCausalLM(nn.Module):
    def __init__(self, model_path, config, precisions=None, torch_dtype=torch.float16, fuse_layers=False,
                 trust_remote_code=True):
        super().__init__()
        from transformers import AutoModelForCausalLM

        if torch_dtype != torch.float16:
            raise RuntimeError("Only float16 is supported for now.")
        if not hasattr(config, "anyprec"):
            raise ValueError("config has no `anyprec` entry: not an any-precision checkpoint")
        if config.anyprec.get("group_count", 1) != 1:
            raise ValueError("only group_count == 1 checkpoints are supported (as in the reference packer)")
        self.config = config
        self.supported_bits = list(range(config.anyprec["seed_precision"], config.anyprec["parent_precision"] + 1))
        if precisions is None:
            self.precisions = self.supported_bits
        else:
            if len(precisions) != len(set(precisions)):
                raise ValueError("Precisions must be unique")
            if not all(bit in self.supported_bits for bit in precisions):
                raise ValueError(f"Supported bits {precisions} must be a subset of model supported bits "
                                 f"{self.supported_bits}")
            self.precisions = list(precisions)
        self.precision = max(self.precisions)

        # the skeleton holds no storage until the checkpoint (or the random init) supplies it
        with torch.device("meta"):
            self.model = AutoModelForCausalLM.from_config(config, dtype=torch_dtype)
        self.model.eval()

        self.ap_linears = []
        self._load_quantized_modules()
        self.tie_weights()
        if model_path is not None:
            self._load_checkpoint(model_path)
            self.prune_precisions()

    # ------------------------------------------------------------------ construction
    @staticmethod
    def _load_config(model_path, trust_remote_code=True):
        from transformers import AutoConfig
        return AutoConfig.from_pretrained(model_path, trust_remote_code=trust_remote_code, local_files_only=True)

    @classmethod
    def from_quantized(cls, quant_model_path, trust_remote_code=True, fuse_layers=False, precisions=None):
        config = cls._load_config(quant_model_path, trust_remote_code)
        return cls(model_path=quant_model_path, precisions=precisions, config=config, fuse_layers=fuse_layers,
                   trust_remote_code=trust_remote_code)

    @classmethod
    def from_config(cls, config, seed=0, device="cuda", precisions=None, std=0.02):
        """A randomly initialised model of the architecture ``config`` describes: embeddings, norms and
        head N(0, std) fp16 (norm weights 1), every listed linear as uniform parent codes with one
        ascending N(0, std) table per row and precision.  ``config.anyprec`` is filled in for a
        Llama-style module layout if absent."""
        if not hasattr(config, "anyprec"):
            config.anyprec = {"seed_precision": 3, "parent_precision": 8, "group_count": 1,
                              "arch_config": dict(LLAMA_ARCH_CONFIG)}
        self = cls(model_path=None, config=config, precisions=precisions)
        gen = torch.Generator(device=device)
        gen.manual_seed(seed)
        ap_ids = {id(m) for m in self.ap_linears}
        for module in self.model.modules():
            if id(module) in ap_ids:
                N, W = module.out_features, module.in_features // 32
                module.qweight = torch.randint(-2**31, 2**31 - 1, (max(self.supported_bits), N, W), dtype=torch.int32,
                                               device=device, generator=gen)
                for b in self.supported_bits:
                    t = torch.randn((N, 1 << b), device=device, generator=gen) * std
                    setattr(module, f"lut{b}", torch.sort(t, dim=1).values.to(torch.float16).contiguous())
                if module.bias is not None:
                    module.bias = torch.zeros((N,), dtype=torch.float16, device=device)
                continue
            for name, p in list(module.named_parameters(recurse=False)):
                if p.ndim == 1:   # norm weights
                    value = torch.ones(p.shape, dtype=p.dtype, device=device)
                else:
                    value = (torch.randn(p.shape, device=device, generator=gen) * std).to(p.dtype)
                module._parameters[name] = nn.Parameter(value, requires_grad=False)
        self._materialise_rotary(device)
        self.tie_weights()
        self.prune_precisions()
        left = [n for n, t in list(self.model.named_parameters()) + list(self.model.named_buffers()) if t.is_meta]
        if left:
            raise RuntimeError(f"no initialiser for {left[:5]}")
        return self

    def _materialise_rotary(self, device):
        """Rotary tables are non-persistent buffers computed in ``__init__``; a meta-device build leaves
        them without storage, so they are recomputed from the config."""
        for module in self.model.modules():
            if hasattr(module, "inv_freq") and module.inv_freq.is_meta:
                with torch.device("cpu"):
                    fresh = type(module)(config=self.config)
                module.inv_freq = fresh.inv_freq.to(device)
                if hasattr(module, "original_inv_freq"):
                    module.original_inv_freq = fresh.inv_freq.to(device)

    def _load_quantized_modules(self):
        arch = self.config.anyprec["arch_config"]
        for layer in self.get_model_layers():
            for name in arch["module_names"]:
                module = _get_by_name(layer, name)
                ap = AnyPrecisionLinear(module.in_features, module.out_features, self.supported_bits,
                                        bias=module.bias is not None, precisions=self.precisions,
                                        device=module.weight.device, dtype=torch.float16)
                self.ap_linears.append(ap)
                _set_by_name(layer, name, ap)

    def _load_checkpoint(self, model_path):
        path = os.path.join(model_path, "pytorch_model.bin")
        state = torch.load(path, map_location="cpu", weights_only=True, mmap=True)
        missing, unexpected = self.model.load_state_dict(state, strict=False, assign=True)
        missing = [k for k in missing if "rotary_emb" not in k and not (k == "lm_head.weight" and
                                                                        getattr(self.config, "tie_word_embeddings", False))]
        if missing or unexpected:
            raise RuntimeError(f"checkpoint does not match the model: missing {missing[:5]}, unexpected {unexpected[:5]}")
        self._materialise_rotary("cpu")
        self.tie_weights()

    def save_quantized(self, output_model_path):
        """Writes the directory the reference packer writes (pack.py:165-177), minus the tokenizer."""
        if set(self.precisions) != set(self.supported_bits):
            # prune_precisions() has dropped planes and tables that config.anyprec still promises
            raise RuntimeError(f"this model was loaded with precisions {self.precisions} of {self.supported_bits} and "
                               "holds only their planes and tables: load it with every precision to save it")
        os.makedirs(output_model_path, exist_ok=True)
        state = {k: v.detach().cpu() for k, v in self.model.state_dict().items()}
        torch.save(state, os.path.join(output_model_path, "pytorch_model.bin"))
        self.config.save_pretrained(output_model_path)

    # ------------------------------------------------------------------ reference surface
    def forward(self, *args, **kwargs):
        prev_precision = self.precision
        if "precision" in kwargs:
            self.set_precision(kwargs.pop("precision"))
        try:
            return self.model.forward(*args, **kwargs)
        finally:
            self.set_precision(prev_precision)

    def generate(self, *args, **kwargs):
        prev_precision = self.precision
        if "precision" in kwargs:
            self.set_precision(kwargs.pop("precision"))
        try:
            with torch.inference_mode():
                return self.model.generate(*args, **kwargs)
        finally:
            self.set_precision(prev_precision)

    def prune_precisions(self):
        for ap_linear in self.ap_linears:
            ap_linear.prune_precisions()
        gc.collect()

    def set_precision(self, precision):
        for ap_linear in self.ap_linears:
            ap_linear.set_precision(precision)
        self.precision = precision

    def tie_weights(self):
        if hasattr(self.model, "tie_weights"):
            self.model.tie_weights()

    def get_model_layers(self):
        arch = self.config.anyprec["arch_config"]
        return _get_by_name(_get_by_name(self.model, arch["model_name"]), arch["layers_name"])

    def fuse_layers(self):
        raise NotImplementedError("This model does not support layer fusion")

    @property
    def layer_type(self):
        for layer in self.get_model_layers():
            if layer.__class__.__name__.endswith("DecoderLayer"):
                return layer.__class__.__name__
        return None

    @property
    def device(self):
        return self.model.device

    # ------------------------------------------------------------------ dense reconstruction
    def dense_state_dict(self, precision):
        """State dict of the plain fp16 model whose linears hold the weights this model uses at
        ``precision`` (one ``dequant_kbit`` per linear, bit-exact table copies)."""
        from any_precision_ext import dequant_kbit
        if precision not in self.precisions:
            raise RuntimeError(f"{self.precisions}-bit precisions are supported but {precision}-bit was specified.")
        out = {}
        ap_names = {id(m): n for n, m in self.model.named_modules() if isinstance(m, AnyPrecisionLinear)}
        skip = tuple(n + "." for n in ap_names.values())
        for key, value in self.model.state_dict().items():
            if not key.startswith(skip):
                out[key] = value
        for module in self.ap_linears:
            name = ap_names[id(module)]
            out[name + ".weight"] = dequant_kbit(module.qweight, module._buffers[f"lut{precision}"], precision)
            if module.bias is not None:
                out[name + ".bias"] = module.bias
        return out

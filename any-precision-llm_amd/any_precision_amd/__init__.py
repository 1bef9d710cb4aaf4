"""Host side of the MI355X any-precision bitplane path.

* ``any_precision_ext`` (sibling top-level module): the drop-in op module.
* ``AnyPrecisionLinear``: counterpart of the reference's operator module.
* ``AnyPrecisionForCausalLM`` (``causal_lm``): counterpart of the reference's model wrapper;
  ``GraphDecoder`` (``decode``): greedy decoding with the step captured in a HIP graph.
* ``packing``: numpy packer/unpacker of the bitplane checkpoint layout.
* ``synth``: seeded synthetic layers of the benchmark configurations.

Importing the ops requires the built HIP library; ``packing`` and ``synth``
are pure numpy and import without it.
"""
from . import packing, synth  # noqa: F401

__all__ = ["packing", "synth", "AnyPrecisionLinear", "AnyPrecisionForCausalLM", "GraphDecoder"]


def __getattr__(name):
    if name == "AnyPrecisionLinear":
        from .linear import AnyPrecisionLinear
        return AnyPrecisionLinear
    if name == "AnyPrecisionForCausalLM":
        from .causal_lm import AnyPrecisionForCausalLM
        return AnyPrecisionForCausalLM
    if name == "GraphDecoder":
        from .decode import GraphDecoder
        return GraphDecoder
    raise AttributeError(name)

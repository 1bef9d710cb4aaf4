"""Host side of the MI355X any-precision bitplane path.

* ``any_precision_ext`` (sibling top-level module): the drop-in op module.
* ``AnyPrecisionLinear``: counterpart of the reference's operator module.
* ``packing``: numpy packer/unpacker of the bitplane checkpoint layout.
* ``synth``: seeded synthetic layers of the benchmark configurations.

Importing the ops requires the built HIP library; ``packing`` and ``synth``
are pure numpy and import without it.
"""
from . import packing, synth  # noqa: F401

__all__ = ["packing", "synth", "AnyPrecisionLinear"]


def __getattr__(name):
    if name == "AnyPrecisionLinear":
        from .linear import AnyPrecisionLinear
        return AnyPrecisionLinear
    raise AttributeError(name)

"""IRON's operator hot path on one AMD Instinct MI355X (gfx950).

Hand-written HIP kernels behind a C ABI (``libiron_hip.so``), the reference's
operator / graph / lm Python API on top.  Host arrays of bf16 operands are
float32 numpy arrays holding bf16-representable values (``iron_amd.bf16``).
"""

from .bf16 import bfloat16, round_bf16  # noqa: F401

__version__ = "0.1.0"


_LAZY = dict.fromkeys(
    ["Carried", "CarriedLoop", "CompiledGraph", "Graph", "Scratchpad", "carry", "clamp", "param", "state", "weight"],
    "iron_amd.common.graph",
) | dict.fromkeys(["Precision"], "iron_amd.common.declare") | dict.fromkeys(["Profile"], "iron_amd.common.profile")


def __getattr__(name):
    import importlib

    module = _LAZY.get(name)
    if module is None:
        raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
    return getattr(importlib.import_module(module), name)

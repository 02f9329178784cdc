"""IRON's operator hot path on one AMD Instinct MI355X (gfx950).

Hand-written HIP kernels behind a C ABI (``libiron_hip.so``), the reference's
operator / graph / lm Python API on top.  Host arrays of bf16 operands are
float32 numpy arrays holding bf16-representable values (``iron_amd.bf16``).
"""

from .bf16 import bfloat16, round_bf16  # noqa: F401

__version__ = "0.1.0"

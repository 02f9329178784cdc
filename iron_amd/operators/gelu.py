"""GELU, by its tanh approximation or exact (iron/operators/gelu.py:13)."""

from __future__ import annotations

from typing import ClassVar

from ..common.declare import Built, param
from ..common.testing import Testing
from ..common.verify import Tolerance
from .elementwise import Sweep, UnaryElementwise


class GELU(UnaryElementwise):
    """``0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3)))``, or exact (``approximate="none"``,
    ``x * Phi(x)``), as torch's ``approximate``."""

    test = Testing([Sweep(), Sweep(approximate="none", bench=None)], draw=lambda op: dict(centered=(op.x,)))
    tile_cap: ClassVar[int] = 8192

    approximate: str = param(default="tanh", array=True)

    def validate(self) -> None:
        if self.approximate not in ("tanh", "none"):
            raise ValueError(f"GELU: approximate={self.approximate!r} is neither 'tanh' nor 'none'")

    def tolerance(self) -> Tolerance:
        # One bf16 step, and what float32 leaves of 1 + tanh / 1 + erf far in the negative tail.
        return Tolerance.relative(2.0**-7, 1e-5, note="f32 math, rounded once")

    def build(self) -> Built:
        from .. import kernels

        n, kind = self.size, "gelu_tanh" if self.approximate == "tanh" else "gelu_erf"

        def launch(t, words):
            kernels.unary(t["x"], t["y"], kind, n=n, valid=words.get("valid"))

        return Built("iron_unary_bf16", launch)

"""Clamp: ``x`` clamped to ``[low, high]``, the bounds rounded to bf16 (iron/operators/clamp.py:14)."""

from __future__ import annotations

import numpy as np

from ..bf16 import round_bf16
from ..common.declare import Built, param
from ..common.testing import Case, Testing
from ..common.verify import Tolerance
from .elementwise import Sweep, UnaryElementwise


class Clamp(UnaryElementwise):
    test = Testing(
        [
            Sweep(low=-0.75, high=1.25),
            # Bounds of one sign, and one past every input: the identity.
            Case(dict(size=2048, low=0.5, high=1.5)),
            Case(dict(size=2048, low=-3e4, high=3e4)),
        ],
        draw=lambda op: dict(centered=(op.x,)),
    )

    low: float = param()
    high: float = param()

    def validate(self) -> None:
        if not np.float32(self.low) <= np.float32(self.high):
            raise ValueError(f"Clamp: low ({self.low}) exceeds high ({self.high})")

    def bounds(self) -> tuple[float, float]:
        """The bounds as the kernel takes them: each rounded to bf16."""
        low, high = round_bf16(np.array([self.low, self.high], np.float32))
        return float(low), float(high)

    def tolerance(self) -> Tolerance:
        return Tolerance.exact(note="a selection")

    def build(self) -> Built:
        from .. import kernels

        n, (low, high) = self.size, self.bounds()

        def launch(t, words):
            kernels.unary(t["x"], t["y"], "clamp", n=n, low=low, high=high, valid=words.get("valid"))

        return Built("iron_unary_bf16", launch)

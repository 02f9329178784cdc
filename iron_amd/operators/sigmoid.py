"""Sigmoid, ``1 / (1 + exp(-x))`` (iron/operators/sigmoid.py"""

from __future__ import annotations

from ..common.declare import Built
from ..common.testing import Testing
from ..common.verify import Tolerance
from .elementwise import Sweep, UnaryElementwise


class Sigmoid(UnaryElementwise):
    test = Testing(Sweep(), draw=lambda op: dict(centered=(op.x,)))  # both signs

    def tolerance(self) -> Tolerance:
        return Tolerance.bf16_ulps(1, note="f32 math, rounded once")

    def build(self) -> Built:
        from .. import kernels

        n = self.size

        def launch(t, words):
            kernels.unary(t["x"], t["y"], "sigmoid", n=n, valid=words.get("valid"))

        return Built("iron_unary_bf16", launch)

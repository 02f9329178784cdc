"""Element-wise multiplication (iron/operators/elementwise_mul.py:11)."""

from __future__ import annotations

from ..common.declare import Built
from ..common.verify import Tolerance
from .elementwise import BinaryElementwise, RowBroadcast


class ElementwiseMul(BinaryElementwise):
    def tolerance(self) -> Tolerance:
        return Tolerance.exact(note="the product of two bf16 is exact in f32: one rounding")

    def build(self) -> Built:
        from .. import kernels

        n = self.size

        def launch(t, words):
            kernels.mul(t["a"], t["b"], t["y"], n=n, valid=words.get("valid"))

        return Built("iron_mul_bf16", launch)


class RowwiseMul(RowBroadcast):
    """Each row times one row, ``x * row`` (iron/operators/elementwise_mul.py:18)."""

    multiply = True

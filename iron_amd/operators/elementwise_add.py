"""Element-wise addition (iron/operators/elementwise_add.py:11)."""

from __future__ import annotations

from ..common.declare import Built
from ..common.verify import Tolerance
from .elementwise import BinaryElementwise, RowBroadcast


class ElementwiseAdd(BinaryElementwise):
    def tolerance(self) -> Tolerance:
        return Tolerance.exact(note="bf16(f32(a) + f32(b))")

    def build(self) -> Built:
        from .. import kernels

        n = self.size

        def launch(t, words):
            kernels.add(t["a"], t["b"], t["y"], n=n, valid=words.get("valid"))

        return Built("iron_add_bf16", launch)


class RowwiseAdd(RowBroadcast):
    """Each row plus one row, ``x + row``: a projection's bias (iron/operators/elementwise_add.py:18)."""

    multiply = False

"""AXPY, ``a * x + y`` with one scalar ``a`` (iron/operators/axpy.py:13)."""

from __future__ import annotations

from ..common.declare import Built, param
from ..common.testing import Case, Testing
from .elementwise import BinaryElementwise, Sweep


class AXPY(BinaryElementwise):
    """``y = bf16(scalar_factor * a + b)``: the product and the sum in float32, one rounding."""

    # A second scalar on one shape, so it is seen to reach the kernel.
    test = Testing([Sweep(scalar_factor=3.0), Case(dict(size=2048, scalar_factor=1.003))])

    scalar_factor: float = param(default=3.0, array=True)

    def scalars(self) -> tuple:
        return (self.scalar_factor,)

    def build(self) -> Built:
        from .. import kernels

        n, a = self.size, float(self.scalar_factor)

        def launch(t, words):
            kernels.axpy(t["a"], t["b"], t["y"], a=a, n=n, valid=words.get("valid"))

        return Built("iron_axpy_bf16", launch)

"""SiLU, ``x * sigmoid(x)`` (iron/operators/silu.py:12)."""

from __future__ import annotations

from ..common.declare import Built
from ..common.testing import Testing
from .elementwise import Sweep, UnaryElementwise


class SiLU(UnaryElementwise):
    test = Testing(Sweep())

    def build(self) -> Built:
        from .. import kernels

        n = self.size

        def launch(t, words):
            kernels.silu(t["x"], t["y"], n=n, valid=words.get("valid"))

        return Built("iron_silu_bf16", launch)

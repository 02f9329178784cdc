"""LayerNorm of each row (beta 0), optionally times a learned weight row (iron/operators/layer_norm.py:10)."""

from __future__ import annotations

from ..common.declare import Built, param
from ..common.verify import Tolerance
from .elementwise import WeightedRowwise


class LayerNorm(WeightedRowwise):
    """``y = bf16(bf16((x - mean) / sqrt(var + epsilon)) * weight)``: one HIP kernel, a row per block."""

    # The epsilon under the root: torch's 1e-5 by default; a model states its own.
    epsilon: float = param(default=1e-5, array=True)

    def scalars(self) -> tuple:
        return (self.epsilon,)

    def tolerance(self) -> Tolerance:
        return Tolerance.relative(1e-2, 1e-2, note="f32 mean and variance, rounded once (twice weighted)")

    def build(self) -> Built:
        from .. import kernels

        rows, cols, eps = self.rows, self.tile_size, float(self.epsilon)

        def launch(t, words):
            kernels.layernorm(t["x"], t.get("weight"), t["y"], rows=rows, cols=cols, eps=eps,
                              valid=words.get("valid"))

        return Built("iron_layernorm_bf16", launch)

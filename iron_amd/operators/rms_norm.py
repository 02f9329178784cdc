"""RMSNorm of each row, optionally times a learned weight row (iron/operators/rms_norm.py:10)."""

from __future__ import annotations

from ..common.declare import Built, param
from ..common.verify import Tolerance
from .elementwise import WeightedRowwise


class RMSNorm(WeightedRowwise):
    """``y = bf16(bf16(x * rsqrt(mean(x^2) + epsilon)) * weight)``: one fused HIP kernel, a row per block."""

    # The epsilon under the root: 1e-5 by default; a model states its own.
    epsilon: float = param(default=1e-5, array=True)

    def scalars(self) -> tuple:
        return (self.epsilon,)

    def tolerance(self) -> Tolerance:
        # The row's sum runs in another order than the reference's and the row is rounded
        # twice when weighted: within two bf16 steps, or the stated bf16 tolerance.
        return Tolerance.relative(1e-2, 1e-2, note="f32 sum of squares, rounded once (twice weighted)")

    def build(self) -> Built:
        from .. import kernels

        rows, cols, eps = self.rows, self.tile_size, float(self.epsilon)

        def launch(t, words):
            kernels.rmsnorm(t["x"], t.get("weight"), t["y"], rows=rows, cols=cols, eps=eps,
                            valid=words.get("valid"))

        return Built("iron_rmsnorm_bf16", launch)

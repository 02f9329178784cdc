"""Softmax of each row over its last axis (iron/operators/softmax.py:62-545).

bf16 logits, or float32 ones with a float32 addend and a soft cap ``cap * tanh(z / cap)``
before the exponentials; a per-call ``length`` takes the first columns of each row and
leaves the rest zero.  The reference's banded variant (``window``, ``period``: a mask its
AIE core computes from the row's position) is not built and is refused.
"""

from __future__ import annotations

from typing import Any

import numpy as np

from ..bf16 import bfloat16
from ..common.declare import Built, In, Operator, Out, param, per_call, tunable
from ..common.testing import Case, Testing
from ..common.verify import Tolerance


def _draw(op) -> dict:
    """The float32 path's logits and addend centred; the bf16 path draws ``[0, scale)``."""
    if op.input_dtype is bfloat16:
        return {}
    return dict(centered=(op.x,) + ((op.addend,) if op.has_addend else ()))


class Softmax(Operator):
    test = Testing(
        [
            Case(dict(rows=32, cols=1024)),
            Case(dict(rows=16, cols=4608)),
            Case(dict(rows=32, cols=32768)),
            Case(dict(rows=4096, cols=512), bench=True),
            Case(dict(rows=32, cols=1024, input_dtype=np.float32)),
            Case(dict(rows=64, cols=1536, input_dtype=np.float32, has_addend=True, soft_cap=50.0)),
        ],
        draw=_draw,
    )

    rows: int = param(array=True)
    cols: int = param()
    num_aie_columns: int = tunable()
    num_channels: int = tunable(default=1)
    block: int = tunable()
    streamed: bool = tunable()
    input_dtype: Any = param(default=bfloat16, repr=False)
    soft_cap: float | None = param(default=None, array=True)
    has_addend: bool = param(default=False)
    window: int | None = param(default=None, array=True)
    period: int | None = param(default=None, array=True)

    # cols, or fewer per call
    length = per_call(bounds=cols)

    x = In(rows, cols, dtype=input_dtype)
    # A float32 row added to x before the cap, such as relative-position logits.
    addend = In(rows, cols, dtype=np.float32, when=has_addend)
    y = Out(rows, cols)

    def validate(self) -> None:
        if self.rows % 16 != 0:
            raise ValueError(f"Softmax: rows ({self.rows}) must be a multiple of 16")
        if self.cols % 16 != 0:
            raise ValueError(f"Softmax: cols ({self.cols}) must be a multiple of 16")
        if self.input_dtype is bfloat16 and (self.soft_cap is not None or self.has_addend
                                             or self.window is not None or self.period is not None):
            raise ValueError("Softmax: soft_cap, addend, window and period are options of the float32 "
                             "input path; pass input_dtype=np.float32")
        if self.window is not None or self.period is not None:
            raise ValueError("Softmax: the banded path (window, period) is not built")
        if self.soft_cap is not None and not self.soft_cap > 0:
            raise ValueError(f"Softmax: soft_cap ({self.soft_cap}) must be positive")

    @classmethod
    def infer(cls, shapes, **kw):
        x = shapes["x"]
        out = dict(rows=int(np.prod(x[:-1])) if len(x) > 1 else 1, cols=x[-1])
        if "addend" in shapes:
            out["has_addend"] = True
        return out

    def ops(self) -> int:
        return self.rows * self.cols

    def tolerance(self) -> Tolerance:
        return Tolerance.relative(1e-2, 1e-3, note="f32 exponentials and sum, rounded once")

    def build(self) -> Built:
        from .. import kernels

        rows, cols, cap = self.rows, self.cols, self.soft_cap

        def launch(t, words):
            kernels.softmax(t["x"], t["y"], rows=rows, cols=cols, addend=t.get("addend"), soft_cap=cap,
                            length=words.get("length"))

        return Built("iron_softmax_bf16", launch)

"""RoPE, rotary position embedding (iron/operators/rope.py:58-191).

``two_halves`` rotates the two halves of each row (Hugging Face's) or, False, interleaved
pairs (Meta's).  ``angles`` is the packed bf16 table, cos and sin interleaved; each angle
row serves ``rows / angle_rows`` consecutive rows.
"""

from __future__ import annotations

import numpy as np

from ..bf16 import round_bf16
from ..common.declare import Built, In, Operator, Out, param, per_call, tunable
from ..common.testing import Case, Testing
from ..common.verify import Tolerance


def _cases(cls, dev=None):
    return [
        Case(dict(rows=32, cols=512, angle_rows=8)),
        Case(dict(rows=32, cols=512, angle_rows=32)),
        Case(dict(rows=32, cols=128, angle_rows=8, two_halves=False)),
        Case(dict(rows=64, cols=128, angle_rows=16), extensive=True),
        # Llama-3.2-1B's decode (q, k) and prompt chunk (q).
        Case(dict(rows=32, cols=64, angle_rows=1)),
        Case(dict(rows=8, cols=64, angle_rows=1)),
        Case(dict(rows=2048 * 32, cols=64, angle_rows=2048), bench=True),
        Case(dict(rows=4096, cols=512, angle_rows=8), bench=True),
        # part of each row turns (a quarter, half): the rest passes through
        Case(dict(rows=64, cols=32, row=128, angle_rows=2)),
        Case(dict(rows=32, cols=32, row=64, angle_rows=1)),
    ]


def _angles(op):
    """A random angle table, cos and sin interleaved, a row per position (rope.py:49-55)."""
    rng = np.random.default_rng(0)
    theta = rng.uniform(-np.pi, np.pi, (op.angle_rows, op.cols // 2))
    table = np.empty((op.angle_rows, op.cols), dtype=np.float32)
    table[:, ::2], table[:, 1::2] = np.cos(theta), np.sin(theta)
    return dict(given={op.angles: round_bf16(table)})


class RoPE(Operator):
    test = Testing(_cases, draw=_angles)

    rows: int = param()
    cols: int = param()
    angle_rows: int = param(default=lambda op: op.rows)  # one row per position
    num_aie_columns: int = tunable()
    two_halves: bool = param(default=True, array=True)
    # The whole row where only its first ``cols`` columns turn (partial rotary: the reference slices
    # them out, rotates and copies back, iron/lm/blocks.py:612-620; here one launch passes the rest on).
    row: int = param(default=lambda op: op.cols)

    x = In(rows, row)
    angles = In(angle_rows, cols)
    y = Out(rows, row)
    # Either row count may be bounded per call: x[:n] and angles[:m].
    valid = per_call(bounds=rows)
    valid_angles = per_call(bounds=angle_rows)

    def validate(self) -> None:
        if not (self.cols % 16 == 0 and self.cols >= 16):
            raise ValueError(f"RoPE: cols ({self.cols}) must be a positive multiple of 16")
        if self.row < self.cols or (self.row - self.cols) % 8:
            raise ValueError(f"RoPE: a row of {self.row} columns of which {self.cols} turn: the rest must be a "
                             "multiple of 8")
        if not (self.angle_rows <= self.rows and self.rows % self.angle_rows == 0):
            raise ValueError(f"RoPE: angle_rows ({self.angle_rows}) must divide rows ({self.rows})")

    @classmethod
    def infer(cls, shapes, **kw):
        x, a = shapes["x"], shapes["angles"]
        if len(x) != 2 or len(a) != 2 or x[1] < a[1]:
            raise ValueError(f"x {x} and angles {a} are (rows, cols) and (angle_rows, cols)")
        return dict(rows=x[0], cols=a[1], angle_rows=a[0], **({} if x[1] == a[1] else {"row": x[1]}))

    def ops(self) -> int:
        return 3 * self.rows * self.cols

    def tolerance(self) -> Tolerance:
        return Tolerance.relative(0.05, note="within one bf16 ulp on the bf16 tables it is given")

    def build(self) -> Built:
        from .. import kernels

        rows, cols, arows, halves, row = self.rows, self.cols, self.angle_rows, self.two_halves, self.row

        def launch(t, words):
            kernels.rope(t["x"], t["angles"], t["y"], rows=rows, cols=cols, angle_rows=arows,
                         two_halves=halves, valid=words.get("valid"), row_cols=row)

        return Built("iron_rope_bf16", launch)

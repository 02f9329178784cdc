"""Copy: an exact data mover between views with per-call offsets and bounds.

The part of the reference's ``Copy`` / ``Gather`` (iron/operators/copy.py:72,546,839-902)
a decoder graph records: embedding rows gathered by ids, a row (or a run of rows) read at
or written to a per-call position (RoPE-table rows, KV-cache writes, the last prompt
row), whole contiguous copies.  Views are contiguous along their rows.
"""

from __future__ import annotations

import math
from typing import Any

from ..bf16 import bfloat16
from ..common.declare import Built, In, Operator, Out, param, per_call
from ..common.testing import Case, Testing
from ..common.verify import Tolerance


class Copy(Operator):
    """``dst = src``; either may be a view a call places (``table[position]``,
    ``cache[start:start+C][:rows]``), ``src`` may be a gather (``table[ids]``)."""

    test = Testing([Case(dict(shape=(64, 2048))), Case(dict(shape=(8, 64)))])

    shape: tuple = param()
    dtype: Any = param(default=bfloat16, repr=False)
    src = In(shape, dtype=dtype)
    dst = Out(shape, dtype=dtype)
    valid = per_call(bounds=None)

    @classmethod
    def infer(cls, shapes, **kw):
        return dict(shape=tuple(shapes["src"]))

    @classmethod
    def call_operands(cls, args, kwargs):
        if not 1 <= len(args) <= 2:
            raise TypeError(f"Copy takes a source and optionally a destination, got {len(args)} operands")
        return {"src": args[0]}, list(args[1:]), dict(kwargs)

    def takes_view(self, name: str) -> bool:
        return True

    def bind_views(self, inputs, outputs):
        return {}

    def output_valid(self, name, inputs):
        src = inputs["src"]
        return {0: src.valid[0]} if 0 in src.valid and len(src.shape) == len(self.shape) else {}

    def ops(self) -> int:
        return 0

    def tolerance(self) -> Tolerance:
        return Tolerance.exact()

    def build(self) -> Built:
        from .. import kernels

        shape = tuple(self.shape)
        elements = math.prod(shape)

        def launch(t, words):
            views = words.get("__views__", {})
            sv, dv = views.get("src"), views.get("dst")
            src, dst = t["src"].reshape(-1), t["dst"].reshape(-1)
            if sv is not None and sv["ids"] is not None:
                row = elements // shape[0]
                table = src[: sv["rows"] * row].view(sv["rows"], row)
                valid = sv["valid"] if sv["valid"] is not None else sv["ids_valid"]
                kernels.gather_rows(table, sv["ids"].reshape(-1), dst[:elements], valid=valid)
                return
            # Row granularity: what a per-call index steps by, else the view's own rows.
            strides = [v["stride"] for v in (sv, dv) if v is not None and v["index"] is not None]
            bounded = [v for v in (sv, dv) if v is not None and v["valid"] is not None]
            if strides:
                row = strides[0]
                if any(s != row for s in strides):
                    raise ValueError("Copy: source and destination step by different rows")
            elif bounded and shape:
                row = elements // shape[0]
            else:
                row = elements
            rows = elements // row
            valid = bounded[0]["valid"] if bounded else None
            s_idx = sv["index"] if sv is not None else None
            d_idx = dv["index"] if dv is not None else None
            s_rows = sv["rows"] if s_idx is not None else rows
            d_rows = dv["rows"] if d_idx is not None else rows
            kernels.copy_rows(src, dst, rows=rows, row_elems=row, src_rows=s_rows, dst_rows=d_rows,
                              src_row=s_idx, dst_row=d_idx, valid=valid)

        return Built("iron_copy_rows", launch)

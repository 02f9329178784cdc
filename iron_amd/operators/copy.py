"""Copy: an exact data mover between views with per-call offsets and bounds.

The part of the reference's ``Copy`` / ``Gather`` (iron/operators/copy.py:72,546,839-902)
a decoder graph records: embedding rows gathered by ids, a row (or a run of rows) read at
or written to a per-call position (RoPE-table rows, KV-cache writes, the last prompt
row), whole contiguous copies.  Views are contiguous along their rows.
"""

from __future__ import annotations

import math
from typing import Any

import numpy as np

from ..bf16 import bfloat16
from ..common.declare import Built, In, Operator, Out, param, per_call, tunable
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


class GatherWords(Operator):
    """The step the reference records ahead of a ``Gather`` whose ids the device itself produced
    (iron/operators/copy.py:380-470).  On the NPU it turns each id into DMA descriptor words.  A HIP
    gather reads ids straight from memory, so here the control words ARE the ids: ``control``'s
    first ``rows`` words receive them unchanged and the rest of the buffer is left alone.  The
    address words of the reference (``base_lo`` / ``base_hi``) are accepted per call and unused."""

    test = Testing([Case(dict(rows=16, table_rows=64, row_bytes=128, words=64))])

    rows: int = param()
    table_rows: int = param(array=True)
    row_bytes: int = param(array=True)
    words: int = param(default=lambda op: op.rows)
    bounded: bool = param(default=False, array=True)

    ids = In(rows, dtype=np.int32)
    control = Out(words, dtype=np.int32)
    base_lo = per_call(bounds=None)
    base_hi = per_call(bounds=None)
    valid_rows = per_call(bounds=rows)

    def validate(self) -> None:
        if not 1 <= self.rows <= self.words:
            raise ValueError(f"GatherWords: rows ({self.rows}) must be from 1 to words ({self.words})")

    def ops(self) -> int:
        return 0

    def tolerance(self) -> Tolerance:
        return Tolerance.exact()

    def build(self) -> Built:
        from .. import kernels

        rows = self.rows

        def launch(t, words):
            kernels.copy_rows(t["ids"].reshape(-1), t["control"].reshape(-1)[:rows], rows=rows, row_elems=1,
                              src_rows=rows, dst_rows=rows, valid=words.get("valid_rows"))

        return Built("iron_copy_rows", launch)


class Gather(Operator):
    """``y[i] = table[control[i]]`` for the first ``valid_rows`` of ``rows`` ids: the reference's
    declared gather (iron/operators/copy.py:72-378), which ``Copy(table[ids])`` records implicitly.
    ``control`` holds the ids in its first ``rows`` words (``GatherWords`` writes them, or the host).
    A row whose id lies outside the table is left as it was.  ``feeds`` (pairs of shim columns on the
    reference's device) is accepted and carried; one launch streams every row here."""

    test = Testing([Case(dict(rows=16, table_rows=64, row=64)), Case(dict(rows=2048, table_rows=4096, row=2048), bench=True)])

    rows: int = param()
    table_rows: int = param()
    row: int = param()
    dtype: Any = param(default=bfloat16, repr=False)
    words: int = param(default=lambda op: op.rows, repr=False)
    feeds: int = tunable(default=1)

    table = In(table_rows, row, dtype=dtype)
    control = In(words, dtype=np.int32)
    y = Out(rows, row, dtype=dtype)
    valid_rows = per_call(bounds=rows)

    def validate(self) -> None:
        if self.rows < 1:
            raise ValueError(f"Gather: rows ({self.rows}) must be at least 1")
        if self.words < self.rows:
            raise ValueError(f"Gather: {self.words} control words do not hold {self.rows} ids")
        itemsize = 2 if self.dtype is bfloat16 else np.dtype(self.dtype).itemsize
        if self.row * itemsize % 4:
            raise ValueError(f"Gather: a row of {self.row} elements of {itemsize} bytes is not whole 32-bit words")

    def word_source(self) -> GatherWords:
        """The step that fills ``control`` from ids made on the device."""
        itemsize = 2 if self.dtype is bfloat16 else np.dtype(self.dtype).itemsize
        return GatherWords(rows=self.rows, table_rows=self.table_rows, row_bytes=self.row * itemsize,
                           words=self.words)

    def ops(self) -> int:
        return 0   # a mover: its figure is bandwidth

    def tolerance(self) -> Tolerance:
        return Tolerance.exact()

    def build(self) -> Built:
        from .. import kernels

        rows = self.rows

        def launch(t, words):
            kernels.gather_rows(t["table"], t["control"].reshape(-1)[:rows], t["y"], valid=words.get("valid_rows"))

        return Built("iron_gather_rows", launch)

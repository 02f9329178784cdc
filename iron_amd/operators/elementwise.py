"""The shared elementwise and rowwise operator templates.

Shapes and names of iron/common/elementwise.py (``Elementwise`` :151, ``UnaryElementwise``
:494, ``BinaryElementwise`` :525, ``Rowwise`` :555, ``WeightedRowwise`` :619): a flat buffer
in lines of ``tile_size`` (the line does not change the math), or ``rows`` rows of
``tile_size`` for a kernel that reduces over its row.  Each is one streaming HIP kernel.
"""

from __future__ import annotations

from typing import ClassVar

from ..common.declare import In, Operator, Out, param, per_call, tunable
from ..common.testing import Case, Testing
from ..common.verify import Tolerance

LENGTHS = (1024, 2048, 4096, 8192)
BENCH_ELEMENTS = 1 << 23


class Sweep:
    """The cases of an elementwise operator: the regular length, the other lengths
    (extensive) and one large tracked case (elementwise.py:44-133, grids dropped)."""

    def __init__(self, lengths=LENGTHS, *, regular=2048, rows=False, bench=BENCH_ELEMENTS, **extra):
        self.lengths, self.regular, self.rows, self.bench, self.extra = tuple(lengths), regular, rows, bench, extra

    def _kwargs(self, length, tile):
        kw = dict(rows=length // tile, tile_size=tile) if self.rows else dict(size=length)
        return {**kw, **self.extra}

    def __call__(self, cls, dev=None):
        cap = cls.tile_cap
        out = [Case(self._kwargs(n, min(n, cap)), extensive=n != self.regular) for n in self.lengths]
        if self.bench is not None:
            out.append(Case(self._kwargs(self.bench, min(4096, cap)), bench=True))
        return out


class Elementwise(Operator):
    num_aie_columns: int = tunable()
    num_channels: int = tunable(default=1)
    tile_size: int = tunable()

    tile_cap: ClassVar[int] = 4096

    def tolerance(self) -> Tolerance:
        # One rounding of an f32 result; a transcendental may land one bf16 step off.
        return Tolerance.bf16_ulps(1, note="f32 math, rounded once")

    def output_shape(self, name, inputs):
        first = next(iter(inputs.values()))
        return first.shape

    def output_valid(self, name, inputs):
        first = next(iter(inputs.values()))
        return {0: first.valid[0]} if 0 in first.valid else {}


class UnaryElementwise(Elementwise):
    """A flat buffer in, a flat buffer of the same size out."""

    test = Testing(Sweep())
    size: int = param()
    valid = per_call(bounds=size)
    x = In(size)
    y = Out(size)

    @classmethod
    def infer(cls, shapes, **kw):
        n = 1
        for s in shapes["x"]:
            n *= s
        return dict(size=n)

    def ops(self) -> int:
        return self.size


class BinaryElementwise(Elementwise):
    """Two flat buffers in, one of the same size out."""

    test = Testing(Sweep())
    size: int = param()
    valid = per_call(bounds=size)
    a = In(size)
    b = In(size)
    y = Out(size)

    @classmethod
    def infer(cls, shapes, **kw):
        n = 1
        for s in shapes["a"]:
            n *= s
        m = 1
        for s in shapes["b"]:
            m *= s
        if n != m:
            raise ValueError(f"a {shapes['a']} and b {shapes['b']} differ in size")
        return dict(size=n)

    def bind_views(self, inputs, outputs):
        # A bound in rows of a 2-D operand is a bound in elements of the flat buffer.
        for h in inputs.values():
            if 0 in h.valid and h.shape:
                return {"valid": h.valid[0] * (h.elements // h.shape[0])}
        return {}

    def ops(self) -> int:
        return self.size


UnaryElementwise.bind_views = BinaryElementwise.bind_views


class Rowwise(Elementwise):
    """``rows`` rows of ``tile_size`` elements in, the same out, one reduction per row."""

    test = Testing(Sweep(rows=True))
    rows: int = param()
    valid = per_call(bounds=rows)
    tile_size: int = param(array=True)
    tile_cap: ClassVar[int] = 8192
    x = In(rows, tile_size)
    y = Out(rows, tile_size)

    @classmethod
    def infer(cls, shapes, **kw):
        x = shapes["x"]
        if len(x) == 1:
            return dict(rows=1, tile_size=x[0])
        rows = 1
        for s in x[:-1]:
            rows *= s
        return dict(rows=rows, tile_size=x[-1])

    def ops(self) -> int:
        return self.rows * self.tile_size


class RowBroadcast(Rowwise):
    """``rows`` rows of ``tile_size`` elements, each met elementwise by the one ``row``
    (iron/common/elementwise.py:797-867; the reference's cut of a wide row into ``segments``
    lines is its cores' memory limit and does not change the sums)."""

    multiply: ClassVar[bool] = False
    tile_cap: ClassVar[int] = 4096
    test = Testing([Sweep(rows=True), Case(dict(rows=64, tile_size=5120), id="wide_row"),
                    Case(dict(rows=8, tile_size=12288), id="wider_row")])

    segments: int = tunable()
    line: int = tunable()
    x = In(Rowwise.rows, Rowwise.tile_size)
    row = In(Rowwise.tile_size, replicate=True)
    y = Out(Rowwise.rows, Rowwise.tile_size)

    def tolerance(self) -> Tolerance:
        return Tolerance.exact(note="bf16(f32(x) op f32(row))")

    def build(self):
        from .. import kernels
        from ..common.declare import Built

        rows, cols, multiply = self.rows, self.tile_size, self.multiply

        def launch(t, words):
            kernels.row_broadcast(t["x"], t["row"], t["y"], rows=rows, cols=cols, multiply=multiply,
                                  valid=words.get("valid"))

        return Built("iron_row_broadcast_bf16", launch)


class WeightedRowwise(Rowwise):
    """A ``Rowwise`` kernel's rows, optionally times a learned ``weight`` row, the row
    rounded to bf16 between the two (elementwise.py:676-682)."""

    weighted_cap: ClassVar[int] = 4096
    test = Testing([Sweep(rows=True), Sweep(rows=True, weighted=True)])

    weighted: bool = param(default=False)
    x = In(Rowwise.rows, Rowwise.tile_size)
    weight = In(Rowwise.tile_size, replicate=True, when=weighted)
    y = Out(Rowwise.rows, Rowwise.tile_size)

    @classmethod
    def infer(cls, shapes, **kw):
        out = Rowwise.infer.__func__(cls, shapes)
        if "weight" in shapes:
            out["weighted"] = True
        return out

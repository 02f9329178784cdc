"""Graphs over operators: record a ``body`` on handles, plan one arena, run on the GPU.

The subset of the reference's graph layer the Llama decoder records
(iron/common/graph/{compiled,record,handle,carried}.py, iron/common/image/allocator.py):

* ``Graph`` subclasses hold ``param`` / ``weight`` / ``state`` leaves and sub-graphs;
  calling a sub-graph inside a body records there.
* ``Handle``: a contiguous view of a buffer with static slicing, ``reshape``, a
  per-call bound (``x[:n]``), a per-call row index (``x[p]``), a fixed-width window
  from a per-call start (``x[s:s+W]``), gather by ids (``table[ids]``), ``x[key] = v``
  (records a ``Copy``) and ``+`` / ``*`` (Elementwise steps).
* ``CarriedLoop``: a version's carried values looped on the device (HIP-graph replays).
* ``Affine``: per-call integer expressions of one value (``position + 1``,
  ``rows * 32``, clamp, ``>> k``), each a word of the device scratchpad.
* ``CompiledGraph``: every version of a graph shares ONE device arena: residents
  (weights, states) at fixed offsets, transients packed by live range.  A version
  without input tensors (the decode step) is captured in a HIP graph whose first node
  re-derives the per-call words on the device and whose last nodes carry
  ``token`` / ``position`` forward, so replays need no host writes.
"""

from __future__ import annotations

import dataclasses
import inspect
import logging
import math
from collections.abc import Mapping
from typing import Any, Generic, TypeVar

import numpy as np

from ..bf16 import bfloat16, from_torch, itemsize, round_bf16, to_bits
from .declare import Operator, Precision, graph_recorder  # noqa: F401

logger = logging.getLogger(__name__)

ALIGNMENT = 256  # bytes; every arena placement is a multiple
T = TypeVar("T")


class Scratchpad(Generic[T]):
    """Annotation of a per-call value the host writes each call."""


class Carried(Generic[T]):
    """Annotation of a per-call value a call hands to the next (``carry``)."""


# --------------------------------------------------------------- expressions


@dataclasses.dataclass(frozen=True)
class Affine:
    """``(clamp(((value * scale + bias) >> down), lo, hi) & mask) + post`` of one per-call value."""

    value: str
    scale: int = 1
    bias: int = 0
    down: int = 0
    lo: int | None = None
    hi: int | None = None
    mask: int = -1  # 2^k - 1: the remainder by 2^k, a ring's row
    post: int = 0   # added after the floor, clamp or remainder

    @property
    def linear(self) -> bool:
        return self.down == 0 and self.lo is None and self.hi is None and self.mask == -1 and self.post == 0

    def record(self) -> list[int]:
        """``{mul, add, shift, lo, hi, mask, post}`` of the device's expression table."""
        big = 2**31 - 1
        return [self.scale, self.bias, self.down, -big - 1 if self.lo is None else self.lo,
                big if self.hi is None else self.hi, self.mask, self.post]

    @property
    def clamped(self) -> bool:
        return self.lo is not None or self.hi is not None

    @property
    def name(self) -> str:
        n = self.value
        if self.scale != 1:
            n += f"_x{self.scale}"
        if self.bias:
            n += f"_{'p' if self.bias > 0 else 'm'}{abs(self.bias)}"
        if self.down:
            n += f"_d{self.down}"
        if self.clamped:
            n += f"_c{'' if self.lo is None else self.lo}_{'' if self.hi is None else self.hi}"
        if self.mask != -1:
            n += f"_r{self.mask + 1}"
        if self.post:
            n += f"_{'p' if self.post > 0 else 'm'}{abs(self.post)}"
        return n

    def evaluate(self, values: Mapping[str, int]) -> int:
        v = (int(values[self.value]) * self.scale + self.bias) >> self.down
        if self.lo is not None:
            v = max(v, self.lo)
        if self.hi is not None:
            v = min(v, self.hi)
        return (v & self.mask) + self.post

    def __mod__(self, c):
        """The remainder by a power of two of a value that is never negative (a ring's row)."""
        if not isinstance(c, (int, np.integer)) or c <= 0 or c & (c - 1):
            raise TypeError(f"{self.name} % {c}: a per-call value's remainder is by a power of two")
        if self.post:
            raise TypeError(f"{self.name} % {c}: a remainder after a later sum is not a per-call expression")
        return dataclasses.replace(self, mask=self.mask & (int(c) - 1))

    def _need_linear(self, what):
        if not self.linear:
            raise TypeError(f"{self.name}: {what} after a floor or clamp is not a per-call expression")

    def __add__(self, c):
        if isinstance(c, Affine):
            if c.value != self.value or not (c.linear and self.linear):
                raise TypeError("per-call expressions of two values do not mix")
            return dataclasses.replace(self, scale=self.scale + c.scale, bias=self.bias + c.bias)
        if not isinstance(c, (int, np.integer)):
            return NotImplemented
        if not self.linear:  # past a floor, clamp or remainder a number is added last
            return dataclasses.replace(self, post=self.post + int(c))
        return dataclasses.replace(self, bias=self.bias + int(c))

    __radd__ = __add__

    def __sub__(self, c):
        if isinstance(c, Affine):
            if not self.linear and dataclasses.replace(c, post=0) == dataclasses.replace(self, post=0):
                return Affine(self.value, scale=0, bias=self.post - c.post)  # a fixed distance
            return self + (c * -1)
        return self + (-int(c))

    def __rsub__(self, c):
        return (self * -1) + int(c)

    def __mul__(self, c):
        if not isinstance(c, (int, np.integer)):
            return NotImplemented
        if c == 1:
            return self
        self._need_linear("*")
        return dataclasses.replace(self, scale=self.scale * int(c), bias=self.bias * int(c))

    __rmul__ = __mul__

    def __floordiv__(self, c):
        if not isinstance(c, (int, np.integer)) or c <= 0:
            raise TypeError(f"{self.name} // {c}: a per-call value is divided by a positive integer")
        if self.clamped or self.mask != -1 or self.post:
            raise TypeError(f"{self.name}: // after a clamp or a remainder is not a per-call expression")
        if self.linear and self.scale % c == 0 and self.bias % c == 0:  # the floor folds (12 heads' rows // 12)
            return dataclasses.replace(self, scale=self.scale // int(c), bias=self.bias // int(c))
        if c & (c - 1):
            raise TypeError(f"{self.name} // {c}: only a power of two divides a per-call value it does not divide evenly")
        return dataclasses.replace(self, down=self.down + int(c).bit_length() - 1)

    def clamp(self, lo=None, hi=None):
        if self.mask != -1 or self.post:
            raise TypeError(f"{self.name}: a clamp after a remainder is not a per-call expression")
        return dataclasses.replace(
            self,
            lo=lo if self.lo is None else (self.lo if lo is None else max(lo, self.lo)),
            hi=hi if self.hi is None else (self.hi if hi is None else min(hi, self.hi)),
        )

    def __bool__(self):
        raise TypeError(f"{self.name} is known per call, not while recording")

    def _refuse(self, *_):
        raise TypeError(f"{self.name}: only + - * // 2^k, % 2^k and clamp build per-call expressions")

    __lt__ = __le__ = __gt__ = __ge__ = __truediv__ = _refuse


def clamp(x, lo=None, hi=None):
    """``x`` held within ``[lo, hi]``: a per-call expression or a number."""
    if isinstance(x, Affine):
        return x.clamp(lo, hi)
    x = x if lo is None else max(x, lo)
    return x if hi is None else min(x, hi)


@dataclasses.dataclass(frozen=True)
class PerCallValue:
    """A declared per-call value of a graph (``body``'s keyword-only parameter)."""

    name: str
    kind: str  # "scratchpad" | "carried"
    default: int | None = None


class Carry(dict):
    """What a call hands the next: ``carry(token=..., position=...)``."""


def carry(**values) -> Carry:
    return Carry(values)


# ------------------------------------------------------------------- leaves


class _Unbound:
    """A ``param`` whose tensor ``load_state_dict`` has yet to bind."""

    def __init__(self, shape, dtype=bfloat16):
        self.shape, self.dtype = tuple(shape), dtype


class Resident:
    """A tensor the arena holds at one fixed offset for every version."""

    kind = "resident"

    def __init__(self, shape, dtype, array=None):
        self.shape, self.dtype, self.array = tuple(shape), dtype, array

    @property
    def nbytes(self) -> int:
        return math.prod(self.shape) * itemsize(self.dtype)

    # A resident reads as a handle on the graph being recorded.
    def _handle(self) -> "Handle":
        recorder = graph_recorder.get()
        if recorder is None:
            raise TypeError(f"a {self.kind} is indexed inside a graph's body")
        return recorder.resident(self)

    def __getitem__(self, key):
        return self._handle()[key]

    def __setitem__(self, key, value):
        self._handle()[key] = value

    def reshape(self, *shape):
        return self._handle().reshape(*shape)


class Param(Resident):
    kind = "param"


class Weight(Resident):
    kind = "weight"


class State(Resident):
    kind = "state"


def param(*shape_or_array, dtype=bfloat16):
    """A weight a checkpoint fills (``param(out, in)``), or one given as an array."""
    if len(shape_or_array) == 1 and isinstance(shape_or_array[0], np.ndarray):
        a = shape_or_array[0]
        return Param(a.shape, dtype, a)
    return _Unbound(shape_or_array, dtype)


def weight(x):
    """A constant the graph holds (an array), or a param read as a table to gather from."""
    if isinstance(x, Resident):
        return x
    if isinstance(x, _Unbound):
        raise TypeError("weight() of a param that was never loaded")
    a = np.asarray(x)
    if a.dtype == np.float32:
        return Weight(a.shape, bfloat16, round_bf16(a))
    return Weight(a.shape, a.dtype.type, a)


def state(shape, dtype=bfloat16):
    """A tensor that persists from call to call (a KV cache), zero at first."""
    if isinstance(shape, int):
        shape = (shape,)
    if dtype is not bfloat16:
        dtype = np.dtype(dtype).type
    return State(tuple(shape), dtype)


def walk(node, path="", seen=None):
    """Yield ``(path, leaf, parent, key)`` for every leaf and sub-graph under ``node``."""
    seen = set() if seen is None else seen
    if isinstance(node, Graph):
        items = [(k, v) for k, v in vars(node).items() if not k.startswith("_")]
    elif isinstance(node, (list, tuple)):
        items = list(enumerate(node))
    elif isinstance(node, dict):
        items = list(node.items())
    else:
        return
    for key, value in items:
        p = f"{path}{key}"
        if isinstance(value, (Resident, _Unbound)):
            yield p, value, node, key
        elif isinstance(value, (Graph, list, tuple, dict)):
            if isinstance(value, Graph):
                if id(value) in seen:
                    continue
                seen.add(id(value))
                yield p, value, node, key
            yield from walk(value, p + ".", seen)


# ------------------------------------------------------------------ buffers


@dataclasses.dataclass(eq=False)
class Buffer:
    name: str
    shape: tuple[int, ...]
    dtype: Any
    kind: str  # input | resident | transient
    source: Any = None  # the Resident behind a resident buffer

    @property
    def elements(self) -> int:
        return math.prod(self.shape)

    @property
    def nbytes(self) -> int:
        return self.elements * itemsize(self.dtype)


@dataclasses.dataclass(frozen=True, eq=False)
class Handle:
    """A contiguous view into a buffer, with what is known only per call."""

    buffer: Buffer
    shape: tuple[int, ...]
    offset: int = 0  # elements, static
    index: Affine | None = None  # per-call start, in units of `index_stride` elements
    index_stride: int = 0
    index_rows: int = 0  # rows the indexed axis has (the limit a call's value is checked by)
    valid: Mapping[int, Affine] = dataclasses.field(default_factory=dict)
    ids: Any = None  # gather: a Handle of int32 ids (rows of `buffer` named per call)

    @classmethod
    def whole(cls, shape, dtype, name, kind, source=None) -> "Handle":
        return cls(Buffer(name, tuple(shape), dtype, kind, source), tuple(shape))

    @property
    def dtype(self):
        return self.buffer.dtype

    @property
    def elements(self) -> int:
        return math.prod(self.shape)

    @property
    def nbytes(self) -> int:
        return self.elements * itemsize(self.dtype)

    def _recorder(self):
        recorder = graph_recorder.get()
        if recorder is None:
            raise TypeError("a handle is computed with inside a graph's body")
        return recorder

    # -- views -------------------------------------------------------------
    def reshape(self, *shape) -> "Handle":
        if len(shape) == 1 and isinstance(shape[0], (tuple, list)):
            shape = tuple(shape[0])
        shape = tuple(int(s) for s in shape)
        if math.prod(shape) != self.elements:
            raise ValueError(f"reshape: {self.shape} does not hold {shape}")
        if self.ids is not None:
            raise TypeError("reshape: a gather is copied before it is reshaped (Copy.step)")
        valid = {}
        if 0 in self.valid:
            old, new = self.shape[0], shape[0]
            n = self.valid[0]
            if new % old == 0:
                valid = {0: n * (new // old)}
            elif old % new == 0 and isinstance(n, Affine):
                valid = {0: n // (old // new)}
            else:
                raise ValueError(f"reshape: a bound on {old} rows does not carry to {new}")
        return dataclasses.replace(self, shape=shape, valid=valid)

    def __getitem__(self, key) -> "Handle":
        if isinstance(key, (Handle, State, Param, Weight)) or (
            isinstance(key, np.ndarray) and key.dtype.kind in "iu"
        ):
            if isinstance(key, Resident):
                key = key._handle()
            if isinstance(key, np.ndarray):
                key = weight(key.astype(np.int32))._handle()
            if self.index is not None or self.ids is not None:
                raise TypeError("gather: from a whole table, not a per-call view")
            valid = {0: key.valid[0]} if 0 in key.valid else {}
            return dataclasses.replace(self, shape=(key.elements, *self.shape[1:]), ids=key, valid=valid,
                                       index_rows=self.shape[0])
        if isinstance(key, tuple):
            raise TypeError("a handle is sliced along its first axis only")
        row = math.prod(self.shape[1:]) if len(self.shape) > 1 else 1
        if isinstance(key, Affine):
            if self.index is not None or self.ids is not None:
                raise TypeError("a per-call view is indexed once")
            return dataclasses.replace(self, shape=self.shape[1:], index=key, index_stride=row,
                                       index_rows=self.shape[0], valid={})
        if isinstance(key, (int, np.integer)):
            k = int(key) + (self.shape[0] if key < 0 else 0)
            if not 0 <= k < self.shape[0]:
                raise IndexError(f"index {key} is outside {self.shape[0]} rows")
            return dataclasses.replace(self, shape=self.shape[1:], offset=self.offset + k * row, valid={})
        if isinstance(key, slice):
            if key.step not in (None, 1):
                raise TypeError("a handle is sliced with unit steps")
            start, stop = key.start, key.stop
            if isinstance(start, Affine) or isinstance(stop, Affine):
                if start is None and isinstance(stop, Affine):  # x[:n] -- a bound
                    if not (stop.linear or stop.clamped):
                        raise TypeError("a bound may only be linear or clamped")
                    return dataclasses.replace(self, valid={**self.valid, 0: stop})
                if isinstance(start, Affine) and isinstance(stop, Affine):  # x[s:s+W] -- a window
                    width = stop - start
                    if width.scale != 0 or width.bias <= 0:
                        raise TypeError("a window from a per-call start has a fixed width")
                    if self.index is not None or self.ids is not None:
                        raise TypeError("a per-call view is indexed once")
                    w = width.bias
                    if w > self.shape[0]:
                        raise IndexError(f"a window of {w} rows is outside {self.shape[0]}")
                    return dataclasses.replace(self, shape=(w, *self.shape[1:]), index=start,
                                               index_stride=row, index_rows=self.shape[0], valid={})
                raise TypeError("slice: a per-call start needs a per-call stop a fixed width on")
            start = 0 if start is None else int(start)
            stop = self.shape[0] if stop is None else int(stop)
            if not 0 <= start <= stop <= self.shape[0]:
                raise IndexError(f"slice [{start}:{stop}] is outside {self.shape[0]} rows")
            valid = dict(self.valid) if start == 0 else {}
            return dataclasses.replace(self, shape=(stop - start, *self.shape[1:]),
                                       offset=self.offset + start * row, valid=valid)
        raise TypeError(f"a handle is not indexed by {type(key).__name__}")

    def __setitem__(self, key, value) -> None:
        from ..operators.copy import Copy

        Copy.step(value, self[key])

    # -- arithmetic ----------------------------------------------------------
    def _binary(self, other, op_name):
        """``self`` met elementwise by an operand of its shape, or -- where ``self`` has two axes or
        more -- by one row of its last axis (iron/common/graph/handle.py:652-676)."""
        from ..operators.elementwise_add import ElementwiseAdd, RowwiseAdd
        from ..operators.elementwise_mul import ElementwiseMul, RowwiseMul

        if isinstance(other, (int, float, np.integer, np.floating)) and not isinstance(other, bool):
            # A number is a constant row in bf16 (iron/common/graph/handle.py:652-661).
            other = _constant_row(float(other), self.shape[-1] if self.shape else 1)
        if isinstance(other, Resident):
            other = other._handle()
        if not isinstance(other, Handle):
            return NotImplemented
        whole, rowwise = (ElementwiseAdd, RowwiseAdd) if op_name == "+" else (ElementwiseMul, RowwiseMul)
        x, y = self, other
        if len(x.shape) == 1 and len(y.shape) > 1:   # a row met by a matrix: commutative
            x, y = y, x
        if len(x.shape) > 1 and tuple(y.shape) == tuple(x.shape[-1:]):
            rows = x.elements // x.shape[-1]
            return rowwise.step(x.reshape(rows, x.shape[-1]), y).reshape(x.shape)
        if y.elements != x.elements:
            raise TypeError(f"{whole.__name__} of {x!r} takes an operand of its shape or a row of "
                            f"{x.shape[-1] if x.shape else 1}, not {list(y.shape)}")
        return whole.step(x, y).reshape(x.shape)

    def __add__(self, other):
        return self._binary(other, "+")

    def __mul__(self, other):
        return self._binary(other, "*")

    __radd__ = __add__
    __rmul__ = __mul__

    def __truediv__(self, other):
        if not isinstance(other, (int, float, np.integer, np.floating)) or isinstance(other, bool):
            raise TypeError(f"{self!r} is divided by a number, not {other!r}")
        return self * (1 / other)


_CONSTANT_ROWS: dict[tuple[float, int], "Weight"] = {}


def _constant_row(value: float, cols: int) -> "Weight":
    """One row of ``cols`` copies of ``value`` in bf16, the same tensor wherever it is asked for."""
    key = (value, cols)
    if key not in _CONSTANT_ROWS:
        _CONSTANT_ROWS[key] = weight(np.full(cols, value, dtype=np.float32))
    return _CONSTANT_ROWS[key]


# ------------------------------------------------------------------ recorder


@dataclasses.dataclass(eq=False)
class Step:
    op: Operator
    inputs: dict[str, Handle]
    outputs: dict[str, Handle]
    values: dict[str, Affine]  # per-call values bound on this step, by the operator's names


@dataclasses.dataclass(frozen=True)
class Limit:
    """A per-call expression and the rows it must stay within, checked before any dispatch."""

    what: str
    expr: Affine
    lo: int
    hi: int  # inclusive
    # A bounded window: the rows a call touches from `expr` on, which must end within `rows`.
    span: Affine | None = None
    rows: int = 0


class Recorder:
    """Collects the steps a body records (the context ``Op.step`` and handles find)."""

    def __init__(self, graph_name: str, profile=None):
        self.graph_name, self.profile = graph_name, profile
        self.steps: list[Step] = []
        self.residents: dict[int, Handle] = {}
        self.limits: list[Limit] = []
        self._transients = 0
        self._token = None

    def __enter__(self):
        self._token = graph_recorder.set(self)
        return self

    def __exit__(self, *exc):
        graph_recorder.reset(self._token)

    def resident(self, r: Resident) -> Handle:
        h = self.residents.get(id(r))
        if h is None:
            h = self.residents[id(r)] = Handle.whole(r.shape, r.dtype, f"{r.kind}{len(self.residents)}",
                                                     "resident", r)
        return h

    def transient(self, shape, dtype, name) -> Handle:
        self._transients += 1
        return Handle.whole(shape, dtype, f"{name}{self._transients}", "transient")

    def as_handle(self, x) -> Handle:
        if isinstance(x, Handle):
            return x
        if isinstance(x, Resident):
            return self.resident(x)
        if isinstance(x, _Unbound):
            raise TypeError("a param was never loaded (load_state_dict)")
        if isinstance(x, np.ndarray):
            return self.resident(weight(x))
        raise TypeError(f"an operand is a handle or a weight, not {type(x).__name__}")

    def call(self, cls_or_op, operands, kwargs) -> Any:
        cls = cls_or_op if isinstance(cls_or_op, type) else type(cls_or_op)
        try:
            return self._call(cls, cls_or_op, operands, kwargs)
        except (ValueError, TypeError) as e:
            shown = ", ".join(str(tuple(getattr(o, "shape", ()))) for o in operands)
            prefix = f"{self.graph_name}: {cls.__name__}({shown}): "
            if str(e).startswith(prefix):
                raise
            raise type(e)(prefix + str(e)) from e

    def _call(self, cls, cls_or_op, operands, kwargs):
        inputs, outs, rest = cls.call_operands(operands, kwargs)
        inputs = {n: self.as_handle(h) for n, h in inputs.items()}
        outs = [self.as_handle(o) for o in outs]
        decl = cls.declaration
        per_call_names = {m.name for m in decl.per_calls}
        values = {k: v for k, v in rest.items() if k in per_call_names}
        fields = {k: v for k, v in rest.items() if k not in per_call_names and v is not None}
        if isinstance(cls_or_op, Operator):
            op = cls_or_op
        else:
            inferred = cls.infer({n: h.shape for n, h in inputs.items()}, **fields)
            if self.profile is not None:
                for k, v in self.profile.lookup(cls, inferred).items():
                    inferred.setdefault(k, v)
            op = cls(**{**inferred, **fields})
        # Bind what the handles know per call: bounds (x[:n]) to the operator's extents.
        bound: dict[str, Affine] = {}
        for k, v in values.items():
            if isinstance(v, (Affine, int, np.integer)):
                bound[k] = v if isinstance(v, Affine) else Affine("__const__", 0, int(v))
        for name, expr in op.bind_views(inputs, outs).items():
            bound.setdefault(name, expr)
        for k, v in bound.items():
            op.use_value(k, v)
        # Operand sizes must be the declared ones, and only an operand that says so may be a view
        # whose rows a call names (the launch would read the buffer from its first row).
        for b in op.inputs:
            h = inputs[b.name]
            if h.elements != b.elements and not op.takes_view(b.name):
                raise ValueError(f"{b.name} takes {b.shape}, got {h.shape}")
            if (h.index is not None or h.ids is not None) and not op.takes_view(b.name):
                raise TypeError(f"{b.name} is a per-call view: Copy.step() it into a tensor of its own first")
        outputs: dict[str, Handle] = {}
        declared_out = op.outputs
        for i, b in enumerate(declared_out):
            if i < len(outs):
                outputs[b.name] = outs[i]
            elif b.fills:  # in-out: written where it is read
                outputs[b.name] = inputs[b.name]
            else:
                h = self.transient(b.shape, b.dtype, cls.__name__.lower())
                seen_as = op.output_shape(b.name, inputs)
                if seen_as is not None:
                    h = dataclasses.replace(h, shape=tuple(seen_as))
                outputs[b.name] = dataclasses.replace(h, valid=op.output_valid(b.name, inputs))
        result = [outputs[b.name] for b in declared_out]
        for b in op.scratch:  # placed in the arena, live over this step only -- or, kept, for good
            if b.kept:
                outputs[b.name] = self.resident(state(b.shape, b.dtype))
            else:
                outputs[b.name] = self.transient(b.shape, b.dtype, f"{cls.__name__.lower()}_{b.name}")
        for name, h in {**inputs, **outputs}.items():
            if h.index is not None:
                width = max(h.elements // h.index_stride, 1)  # rows the view spans
                if 0 in h.valid:  # only the bounded rows are touched
                    self.limits.append(Limit(f"{cls.__name__}.{name}", h.index, 0, h.index_rows - 1,
                                             span=h.valid[0], rows=h.index_rows))
                else:
                    self.limits.append(Limit(f"{cls.__name__}.{name}", h.index, 0, h.index_rows - width))
            if 0 in h.valid:
                self.limits.append(Limit(f"{cls.__name__}.{name}[:n]", h.valid[0], 0, h.shape[0]))
        self.steps.append(Step(op, inputs, outputs, bound))
        return result[0] if len(result) == 1 else tuple(result)


# ---------------------------------------------------------------- the graph


class Graph:
    """A graph: a subclass whose ``body`` is recorded on handles.

    ``body``'s positional parameters are the inputs (one defaulting to None may be
    left out), its keyword-only ones the per-call values (annotated ``Scratchpad`` or
    ``Carried``), its return the outputs, optionally ending in ``carry(...)``.
    Called in another graph's body, it records there.
    """

    profile = None

    def body(self, *inputs, **values):
        raise NotImplementedError(f"{type(self).__name__} defines no body()")

    @property
    def name(self) -> str:
        return type(self).__name__

    def __call__(self, *args, **kwargs):
        if graph_recorder.get() is None:
            raise TypeError(f"{self.name}: called outside a graph's body; compile() a version to run it")
        return self.body(*args, **kwargs)

    # -- parameters ----------------------------------------------------------
    def _parameters(self):
        sig = inspect.signature(type(self).body)
        hints = {}
        try:
            hints = inspect.get_annotations(type(self).body, eval_str=True)
        except Exception:  # annotations that do not evaluate name no per-call kind
            hints = getattr(type(self).body, "__annotations__", {})
        inputs, optional, values = [], set(), {}
        for p in list(sig.parameters.values())[1:]:
            if p.kind in (p.POSITIONAL_ONLY, p.POSITIONAL_OR_KEYWORD):
                inputs.append(p.name)
                if p.default is None:
                    optional.add(p.name)
            elif p.kind == p.KEYWORD_ONLY:
                ann = hints.get(p.name)
                origin = getattr(ann, "__origin__", None)
                kind = "carried" if origin is Carried else "scratchpad"
                default = None if p.default is inspect.Parameter.empty else int(p.default)
                values[p.name] = PerCallValue(p.name, kind, default)
        return inputs, optional, values

    def held(self) -> dict[int, tuple[str, Resident]]:
        held = {}
        for path, x, _, _ in walk(self):
            if isinstance(x, _Unbound):
                raise TypeError(f"{self.name}: {path} was never loaded")
            if isinstance(x, Resident):
                held.setdefault(id(x), (path, x))
        return held

    def load_state_dict(self, tree: Mapping[str, np.ndarray], *, path: str = "") -> None:
        """Bind each ``param`` held, at any depth, to its tensor in ``tree`` (by dotted path)."""
        if path and not path.endswith("."):
            raise ValueError(f"{self.name}: load_state_dict's path {path!r} must end in a dot")
        if vars(self).get("_bound"):
            raise ValueError(f"{self.name}: already loaded")
        tied: dict[int, list[str]] = {}
        params: dict[str, _Unbound] = {}
        for n, p, _, _ in walk(self):
            if isinstance(p, _Unbound):
                tied.setdefault(id(p), []).append(path + n)
                params.setdefault(tied[id(p)][0], p)
        held = {n for paths in tied.values() for n in paths}
        tensors = {n: t for n, t in tree.items() if n.startswith(path)}
        missing = sorted(params.keys() - tensors.keys())
        extra = sorted(tensors.keys() - held)
        shapes = [f"{n} {tuple(np.shape(tensors[n]))}, not {p.shape}" for n, p in params.items()
                  if n in tensors and tuple(np.shape(tensors[n])) != p.shape]
        if missing or extra or shapes:
            found = {"missing": missing, "extra": extra, "wrong shape": shapes}
            raise ValueError(f"{self.name}: cannot load: "
                             + "; ".join(f"{k} {', '.join(v)}" for k, v in found.items() if v))
        bound: dict[int, Param] = {}
        for paths in tied.values():
            p = params[paths[0]]
            a = tensors[paths[0]]
            if _is_torch(a):  # a bf16 tensor (host or device) is taken as it is
                want = "torch.bfloat16" if p.dtype is bfloat16 else f"torch.{np.dtype(p.dtype).name}"
                if str(a.dtype) != want:
                    raise ValueError(f"{self.name}: cannot load: wrong kind {paths[0]} {a.dtype}, not {want}")
            else:
                a = np.asarray(a)
                a = round_bf16(a) if p.dtype is bfloat16 else a.astype(p.dtype)
            bound_param = Param(p.shape, p.dtype, a)
            for n, x, parent, key in walk(self):
                if x is p:
                    if isinstance(parent, (list, dict)):
                        parent[key] = bound_param
                    else:
                        setattr(parent, key, bound_param)
            bound[id(p)] = bound_param
        self._bound = True

    # -- versions ------------------------------------------------------------
    def record(self, **shapes) -> "Recording":
        """Run ``body`` on handles of the given input shapes (``name=(shape, dtype)``)."""
        inputs, optional, values = self._parameters()
        shapes = {k: v for k, v in shapes.items() if v is not None}
        missing = [p for p in inputs if p not in shapes and p not in optional]
        unknown = [k for k in shapes if k not in inputs]
        if missing or unknown:
            raise TypeError(f"{self.name}: shapes for {missing} missing"
                            + (f"; {unknown} are not inputs" if unknown else ""))
        handles, args = [], []
        for name in inputs:
            if name not in shapes:
                args.append(None)
                continue
            shape, dtype = shapes[name]
            handles.append(Handle.whole(tuple(shape), dtype, name, "input"))
            args.append(handles[-1])
        self.held()  # every param loaded
        with Recorder(self.name, self.profile) as recorder:
            result = self.body(*args, **{v.name: Affine(v.name) for v in values.values()})
        if result is None:
            items = []
        elif isinstance(result, (tuple, list)):
            items = list(result)
        else:
            items = [result]
        carried = None
        if items and isinstance(items[-1], Carry):
            carried = items.pop()
            unknown = [k for k in carried if k not in values or values[k].kind != "carried"]
            if unknown:
                raise TypeError(f"{self.name}: carry() names {unknown}, which body does not take as Carried")
        outputs = [recorder.as_handle(o) for o in items]
        return Recording(self.name, handles, outputs, list(values.values()), carried, recorder.steps,
                         recorder.residents, recorder.limits)

    def compile(self, *, arena: "ScratchArena | None" = None, capture: bool | None = None, check: bool = False,
                full_elf: bool | None = None, fuse: bool = True, **shapes) -> "CompiledGraph":
        """Record a version and plan it into this graph's arena.

        ``capture``: replay the version as one HIP graph (default: when it takes no
        input tensor); ``full_elf`` is the reference's name for the same choice.
        ``check``: judge every step against its operator's ``reference()`` as it runs.
        """
        if capture is None:
            capture = full_elf
        recording = self.record(**shapes)
        arena = arena if arena is not None else self.arena
        version = CompiledGraph(self, recording, arena, capture=capture, check=check, fuse=fuse)
        self._versions.append(version)
        return version

    @property
    def _versions(self) -> list:
        return vars(self).setdefault("_versions_list", [])

    @property
    def versions(self) -> list:
        return list(self._versions)

    @property
    def arena(self) -> "ScratchArena":
        return vars(self).setdefault("_arena_object", ScratchArena())

    def release(self) -> None:
        for v in self._versions:
            v.release()
        self._versions.clear()
        vars(self).pop("_arena_object", None)

    def reference(self, *tensors, **values):
        """Run the body on the host, each step through its operator's ``reference()``."""
        inputs, optional, declared = self._parameters()
        given = dict(zip(inputs, tensors))
        shapes = {n: (np.shape(t), _host_dtype(t)) for n, t in given.items() if t is not None}
        key = tuple((n, s, str(d)) for n, (s, d) in shapes.items())
        cache = vars(self).setdefault("_references", {})
        recording = cache.get(key)
        if recording is None:
            recording = cache[key] = self.record(**shapes)
        values = {**{v.name: v.default for v in declared.values() if v.default is not None}, **values}
        return recording.reference({n: np.asarray(t) for n, t in given.items() if t is not None}, values)


def _is_torch(x) -> bool:
    return type(x).__module__.startswith("torch")


def _host_dtype(t):
    a = np.asarray(t)
    return bfloat16 if a.dtype == np.float32 else a.dtype.type


# --------------------------------------------------------------- recording


class Recording:
    """The steps one version runs, its buffers, and a host ``reference()`` of them."""

    def __init__(self, name, inputs, outputs, values, carried, steps, residents, limits):
        self.name, self.inputs, self.outputs = name, inputs, outputs
        self.values, self.carry, self.steps = values, carried, steps
        self.residents, self.limits = residents, limits

    def check_values(self, values: Mapping[str, int]) -> dict[str, int]:
        known = {v.name for v in self.values}
        unknown = sorted(set(values) - known)
        missing = sorted(v.name for v in self.values if v.name not in values and v.default is None)
        if unknown or missing:
            raise TypeError(f"{self.name}: per-call values {missing} missing"
                            + (f"; {unknown} are not per-call values" if unknown else ""))
        full = {v.name: int(values.get(v.name, v.default)) for v in self.values}
        full["__const__"] = 0
        # The layers of a decoder record the same limits over and over: each distinct one is checked
        # once (the first of its kind names it in a refusal).
        distinct = vars(self).get("_distinct_limits")
        if distinct is None or distinct[0] != len(self.limits):
            seen = {}
            for lim in self.limits:
                seen.setdefault((lim.expr, lim.lo, lim.hi, lim.span, lim.rows), lim)
            distinct = self._distinct_limits = (len(self.limits), list(seen.values()))
        for lim in distinct[1]:
            got = lim.expr.evaluate(full)
            if not lim.lo <= got <= lim.hi:
                raise IndexError(f"{self.name}: {lim.what} = {got} ({lim.expr.name}) is outside "
                                 f"[{lim.lo}, {lim.hi}]")
            if lim.span is not None and got + lim.span.evaluate(full) > lim.rows:
                raise IndexError(f"{self.name}: {lim.what}: {lim.span.evaluate(full)} rows from {got} "
                                 f"({lim.expr.name}) end outside {lim.rows}")
        return full

    def transients(self, runs=()) -> list[tuple[Buffer, int, int]]:
        """Each transient buffer with the first and last step that touches it.

        ``runs``: ``(first, last)`` step ranges launched as one kernel each; a buffer touched
        inside a run is live across the whole run (its last step's output is written while its
        first step's input is still being read).
        """
        run_of = {}
        for first, last in runs:
            for i in range(first, last + 1):
                run_of[i] = (first, last)
        spans: dict[int, list] = {}
        for i, step in enumerate(self.steps):
            lo, hi = run_of.get(i, (i, i))
            for h in (*step.inputs.values(), *step.outputs.values()):
                for b in [h.buffer] + ([h.ids.buffer] if h.ids is not None else []):
                    if b.kind == "transient":
                        span = spans.setdefault(id(b), [b, lo, hi])
                        span[1], span[2] = min(span[1], lo), max(span[2], hi)
        for h in self.outputs:  # an output lives to the end
            if id(h.buffer) in spans:
                spans[id(h.buffer)][2] = len(self.steps)
        return [tuple(s) for s in spans.values()]

    # -- host reference ------------------------------------------------------
    def reference(self, given: Mapping[str, np.ndarray], values: Mapping[str, int]):
        """Run every step through its operator's ``reference()`` on host arrays
        (record.py:340-448): states persist in ``Resident.host``; results are written
        back over the valid rows only."""
        full = self.check_values(values)
        host: dict[int, np.ndarray] = {}

        def array_of(b: Buffer) -> np.ndarray:
            if id(b) in host:
                return host[id(b)]
            if b.kind == "resident":
                r = b.source
                if getattr(r, "host", None) is None:
                    init = r.array if r.array is not None else np.zeros(r.shape, _np_dtype(r.dtype))
                    if _is_torch(init):
                        init = from_torch(init)
                    r.host = np.array(init, dtype=_np_dtype(r.dtype)).reshape(-1)
                host[id(b)] = r.host
            elif b.kind == "input":
                host[id(b)] = np.array(given[b.name], dtype=_np_dtype(b.dtype)).reshape(-1)
            else:
                host[id(b)] = np.zeros(b.elements, _np_dtype(b.dtype))
            return host[id(b)]

        def start_of(h: Handle) -> int:
            return h.offset + (h.index.evaluate(full) * h.index_stride if h.index is not None else 0)

        def read(h: Handle) -> np.ndarray:
            flat = array_of(h.buffer)
            if h.ids is not None:
                ids = read(h.ids).reshape(-1).astype(np.int64)
                row = math.prod(h.shape[1:]) if len(h.shape) > 1 else 1
                table = flat[h.offset : h.offset + h.index_rows * row].reshape(h.index_rows, row)
                n = h.valid[0].evaluate(full) if 0 in h.valid else len(ids)
                out = np.zeros((len(ids), row), flat.dtype)
                out[:n] = table[ids[:n]]
                return out.reshape(h.shape)
            s = start_of(h)
            got = flat[s : s + h.elements]
            if got.size < h.elements:
                # A fixed-width window from a per-call start may run past its buffer; its bound (checked
                # before dispatch) keeps every row that is read inside.  The rest read as zeros here.
                got = np.concatenate([got, np.zeros(h.elements - got.size, flat.dtype)])
            return got.reshape(h.shape)

        def write(h: Handle, value: np.ndarray, rows: int | None) -> None:
            flat = array_of(h.buffer)
            s = start_of(h)
            value = np.asarray(value).reshape(h.shape) if h.shape else np.asarray(value).reshape(())
            if rows is None or not h.shape:
                flat[s : s + h.elements] = value.reshape(-1)
            else:
                row = h.elements // h.shape[0]
                flat[s : s + rows * row] = value.reshape(h.shape[0], -1)[:rows].reshape(-1)

        for step in self.steps:
            op = step.op
            extents = {}
            others = {}
            for k, expr in step.values.items():
                member = next(m for m in op.declaration.per_calls if m.name == k)
                (extents if member.bounds is not None else others)[k] = expr.evaluate(full)
            at = op._at_extents(**extents) if extents else op
            ins = {n: read(h) for n, h in step.inputs.items()}
            results = at._call_reference(ins, values=others)
            for n, h in step.outputs.items():
                if n not in results:  # scratch memory: nothing a reference writes
                    continue
                rows = h.valid[0].evaluate(full) if 0 in h.valid else None
                write(h, results[n], rows)
        outs = []
        for h in self.outputs:
            a = read(h).copy()
            if 0 in h.valid:
                a = a[: h.valid[0].evaluate(full)]
            outs.append(a)
        carried = None
        if self.carry is not None:
            carried = {}
            for k, v in self.carry.items():
                if isinstance(v, Handle):
                    carried[k] = int(read(v).reshape(-1)[0])
                elif isinstance(v, Affine):
                    carried[k] = v.evaluate(full)
                else:
                    carried[k] = int(v)
        return outs, carried


def _np_dtype(dtype):
    return np.float32 if dtype is bfloat16 else np.dtype(dtype)


# -------------------------------------------------------------- arena plan


@dataclasses.dataclass(frozen=True)
class LiveRange:
    """A transient's size and the steps it is live over (inclusive)."""

    nbytes: int
    first: int
    last: int


class Pool:
    """First-fit placement of live ranges: two placements overlap in bytes only if
    their ranges do not overlap in time (iron/common/image/allocator.py:143)."""

    def __init__(self, alignment: int = ALIGNMENT):
        self.alignment = alignment
        self.placed: list[tuple[int, int, LiveRange]] = []  # (offset, end, range)
        self.size = 0

    def place(self, r: LiveRange) -> int:
        size = -(-max(r.nbytes, 1) // self.alignment) * self.alignment
        busy = sorted((o, e) for o, e, p in self.placed if not (p.last < r.first or r.last < p.first))
        offset = 0
        for o, e in busy:
            if offset + size <= o:
                break
            offset = max(offset, e)
        self.placed.append((offset, offset + size, r))
        self.size = max(self.size, offset + size)
        return offset


class ScratchArena:
    """One device allocation for every version of a graph: residents at fixed offsets
    (laid out once, shared by all versions), then a transient region as large as the
    largest version needs (iron/common/image/callable.py:68, allocator.py:175-227)."""

    def __init__(self, alignment: int = ALIGNMENT):
        self.alignment = alignment
        self.resident_offsets: dict[int, int] = {}
        self.residents: dict[int, Resident] = {}
        self.resident_bytes = 0
        self.transient_bytes = 0
        self.buffer = None  # torch.uint8 on the GPU
        self.uploaded: set[int] = set()
        self.generation = 0

    def place_resident(self, r: Resident) -> int:
        if id(r) not in self.resident_offsets:
            if self.buffer is not None:
                raise RuntimeError("the arena is loaded: compile every version before load()")
            self.resident_offsets[id(r)] = self.resident_bytes
            self.residents[id(r)] = r
            self.resident_bytes += -(-r.nbytes // self.alignment) * self.alignment
        return self.resident_offsets[id(r)]

    def reserve_transients(self, nbytes: int) -> None:
        if nbytes > self.transient_bytes:
            if self.buffer is not None:
                raise RuntimeError("the arena is loaded: compile every version before load()")
            self.transient_bytes = nbytes

    @property
    def nbytes(self) -> int:
        return self.resident_bytes + self.transient_bytes

    def load(self, device="cuda") -> None:
        """Allocate the arena and upload every resident once."""
        import torch

        if self.buffer is None:
            logger.info("arena: %.1f MB residents + %.1f MB transients", self.resident_bytes / 1e6,
                        self.transient_bytes / 1e6)
            self.buffer = torch.zeros(max(self.nbytes, self.alignment), dtype=torch.uint8, device=device)
            self.generation += 1
        for key, r in self.residents.items():
            if key in self.uploaded:
                continue
            if r.array is not None:
                self.view(self.resident_offsets[key], r.shape, r.dtype).copy_(_host_tensor(r.array, r.dtype))
            self.uploaded.add(key)

    def view(self, offset: int, shape, dtype):
        import torch

        tdtype = torch.bfloat16 if dtype is bfloat16 else getattr(torch, np.dtype(dtype).name)
        n = math.prod(shape) * itemsize(dtype)
        return self.buffer[offset : offset + n].view(tdtype).view(tuple(shape) or (1,))

    def release(self) -> None:
        self.buffer = None
        self.uploaded.clear()


def _host_tensor(array, dtype):
    import torch

    if isinstance(array, torch.Tensor):
        return array
    if dtype is bfloat16:
        return torch.from_numpy(to_bits(array).view(np.int16)).view(torch.bfloat16)
    return torch.from_numpy(np.ascontiguousarray(array, dtype=dtype))


# ------------------------------------------------------------ compiled graph

WORD_SLOTS = 64  # int32 words of the per-call scratchpad
EXPR_WORDS = 9  # int32 words of one record of the device's expression table


class DeviceOutput:
    """An output buffer on the device; ``numpy()`` reads it back (bf16 as float32 values)."""

    def __init__(self, tensor, valid_rows=None):
        self.tensor, self.valid_rows = tensor, valid_rows

    def numpy(self) -> np.ndarray:
        a = from_torch(self.tensor)
        return a if self.valid_rows is None else a[: self.valid_rows]


class CompiledGraph:
    """One version of a graph, placed in its arena; call it with tensors and per-call values."""

    def __init__(self, graph: Graph, recording: Recording, arena: ScratchArena, *, capture=None, check=False,
                 fuse=True):
        self.graph, self.recording, self.arena = graph, recording, arena
        self.check = check
        # Launch the runs of one-row steps a decoder layer records together as fused kernels.
        self.fuse = fuse and not check
        self._fused: dict[int, Any] = {}
        self.capture = (not recording.inputs) if capture is None else bool(capture)
        if check:
            self.capture = False
        # Residents first (fixed for every version), then this version's transients.
        for h in recording.residents.values():
            arena.place_resident(h.buffer.source)
        pool = Pool(arena.alignment)
        self.transient_offsets: dict[int, int] = {}
        # Inputs are transients that live from the start.
        for h in recording.inputs:
            self.transient_offsets[id(h.buffer)] = pool.place(LiveRange(h.buffer.nbytes, -1, len(recording.steps)))
        runs = []
        if self.fuse:
            from . import fusion

            matched = fusion.match(recording)
            runs = [(f.first, f.first + f.count - 1) for f in matched]
        for b, first, last in recording.transients(runs):
            self.transient_offsets[id(b)] = pool.place(LiveRange(b.nbytes, first, last))
        # Memory a fused run needs for itself (partial sums), live over its steps, by the run's first step.
        self.scratch_offsets: dict[int, int] = {}
        if self.fuse:
            for f in matched:
                if f.scratch_bytes:
                    self.scratch_offsets[f.first] = pool.place(LiveRange(f.scratch_bytes, f.first, f.first + f.count - 1))
        # The per-call words: one slot per declared value, then one per derived expression.
        self.slots: dict[str, int] = {v.name: i for i, v in enumerate(recording.values)}
        self.exprs: dict[Affine, int] = {}
        for step in recording.steps:
            for expr in step.values.values():
                self._slot(expr)
            for h in (*step.inputs.values(), *step.outputs.values()):
                if h.index is not None:
                    self._slot(h.index)
                if 0 in h.valid:
                    self._slot(h.valid[0])
                if h.ids is not None and 0 in h.ids.valid:
                    self._slot(h.ids.valid[0])
        if len(self.slots) + len(self.exprs) > WORD_SLOTS:
            raise ValueError(f"{graph.name}: more than {WORD_SLOTS} per-call words")
        # The words and the expression table outlive a call (a replay starts from the last
        # one's values; the table is written once), so they are residents of this version.
        self._words_resident = State((WORD_SLOTS * (1 + EXPR_WORDS),), np.int32)
        arena.place_resident(self._words_resident)
        arena.reserve_transients(pool.size)
        self._loaded_generation = None
        self._graph = None
        self._graph_bounded = None
        # What a step's launch may read of the call's context: ``bounded`` while every step that has a
        # cheaper form within a limit (``Built.bounded``) is being launched, or captured, in that form.
        self._context: dict[str, Any] = {"bounded": False}
        self._bounds: list[tuple[Affine, int]] = []   # (per-call expression, limit) of those steps
        self._launches: list = []

    def _slot(self, expr: Affine) -> int:
        if expr.value in self.slots and expr == Affine(expr.value):
            return self.slots[expr.value]
        if expr not in self.exprs:
            self.exprs[expr] = len(self.slots) + len(self.exprs)
        return self.exprs[expr]

    # -- loading -------------------------------------------------------------
    def _scratch(self, first: int, nbytes: int):
        """The float32 words placed for the fused run that starts at step ``first``."""
        return self.arena.view(self.arena.resident_bytes + self.scratch_offsets[first], (nbytes // 4,), np.float32)

    def _tensor(self, h: Handle):
        b = h.buffer
        if b.kind == "resident":
            base = self.arena.resident_offsets[id(b.source)]
        else:
            base = self.arena.resident_bytes + self.transient_offsets[id(b)]
        whole = self.arena.view(base, (b.elements,), b.dtype)
        if h.index is not None or h.ids is not None:
            return whole[h.offset :]  # the rest of the buffer: the kernel adds the per-call rows
        return whole[h.offset : h.offset + h.elements].view(h.shape or (1,))

    def word(self, expr: Affine | None):
        """The 1-element device view of the scratchpad word holding ``expr``."""
        if expr is None:
            return None
        i = self._slot(expr)
        return self.words[i : i + 1]

    def load(self) -> "CompiledGraph":
        """Bind this version to the loaded arena: tensor views, words, launches, HIP graph."""
        import torch

        self.arena.load()
        if self._loaded_generation == self.arena.generation:
            return self
        base = self.arena.resident_offsets[id(self._words_resident)]
        self.words = self.arena.view(base, (WORD_SLOTS,), np.int32)
        self.expr_table = self.arena.view(base + WORD_SLOTS * 4, (WORD_SLOTS * EXPR_WORDS,), np.int32)
        self.host_words = torch.zeros(WORD_SLOTS, dtype=torch.int32).pin_memory()
        self._host_words_np = self.host_words.numpy()   # the same pinned memory
        self._staging: dict[int, Any] = {}              # per input: a pinned buffer and its copy's event
        # Device-side expression table: derived words, then the carried values.
        rows = []
        big = 2**31 - 1
        for expr, slot in self.exprs.items():
            src = self.slots.get(expr.value)
            if expr.value == "__const__":
                src, expr = 0, dataclasses.replace(expr, scale=0)
            rows.append([slot, src, *expr.record()])
        self.n_derived = len(rows)
        carried = self.recording.carry or {}
        self.carry_copies = []  # (value slot, handle) for values carried from a device buffer
        for k, v in carried.items():
            if isinstance(v, Affine):
                rows.append([self.slots[k], self.slots[v.value], *v.record()])
            elif isinstance(v, Handle):
                self.carry_copies.append((self.slots[k], v))
            else:
                rows.append([self.slots[k], 0, 0, int(v), 0, -big - 1, big, -1, 0])
        self.n_exprs = len(rows)
        # A replay ends by carrying its values and re-deriving the words the next replay reads, in
        # one launch: the carried rows are followed by a second copy of the derived ones.
        self.n_tail = 0
        if self.n_exprs > self.n_derived and self.n_exprs + self.n_derived <= WORD_SLOTS:
            rows = rows + rows[: self.n_derived]
            self.n_tail = self.n_exprs
        if rows:
            table = torch.tensor(rows, dtype=torch.int32).reshape(-1)
            self.expr_table[: table.numel()].copy_(table)
        # A value carried from the draw's own output is written into its word by the draw itself.
        self._carry_by_draw: dict[int, int] = {}
        last = self.recording.steps[-1] if self.recording.steps else None
        if last is not None and type(last.op).__name__ == "Sample":
            for slot, h in list(self.carry_copies):
                if h.buffer is last.outputs["token"].buffer and h.offset == last.outputs["token"].offset:
                    self._carry_by_draw[len(self.recording.steps) - 1] = slot
                    self.carry_copies.remove((slot, h))
        # ... and where the draw is the captured step's last launch and nothing else is carried from a
        # buffer, it evaluates the tail's expressions too: the step ends without a launch for them.
        self._tail_in_draw = bool(self.capture and self._carry_by_draw and self.n_tail and not self.carry_copies)
        self._bounds = []
        self._launches = [self._bind(step) for step in self.recording.steps]
        self._fused = {}
        if self.fuse:
            from . import fusion

            self._fused = {f.first: f for f in fusion.plan(self.recording, self._tensor, self.word, self._scratch)}
        self.input_tensors = [self._tensor(h) for h in self.recording.inputs]
        self.output_tensors = [self._tensor(h) for h in self.recording.outputs]
        self._loaded_generation = self.arena.generation
        self._graph = self._graph_bounded = None
        if self.capture:
            self._capture()
        return self

    def _bind(self, step: Step):
        built = step.op.compile()
        tensors = {n: self._tensor(h) for n, h in {**step.inputs, **step.outputs}.items()}
        words = {k: self.word(e) for k, e in step.values.items()}
        views = {}
        for n, h in {**step.inputs, **step.outputs}.items():
            if h.index is not None or h.ids is not None or 0 in h.valid:
                views[n] = dict(
                    index=self.word(h.index), ids=None if h.ids is None else self._tensor(h.ids),
                    ids_valid=self.word(h.ids.valid.get(0)) if h.ids is not None else None,
                    valid=self.word(h.valid.get(0)), rows=h.index_rows, stride=h.index_stride,
                )
        if views:
            words = {**words, "__views__": views}
        if built.bounded is not None and built.bounded[0] in step.values:
            self._bounds.append((step.values[built.bounded[0]], int(built.bounded[1])))
            words = {**words, "__context__": self._context}
        slot = self._carry_by_draw.get(self.recording.steps.index(step)) if self._carry_by_draw else None
        if slot is not None:
            words = {**words, "__carry_token__": self.words[slot : slot + 1]}
            if self._tail_in_draw:
                words["__carry_eval__"] = (self.words, self.expr_table[EXPR_WORDS * self.n_derived :], self.n_tail)
        return built.launch, tensors, words

    def _run_steps(self) -> None:
        i, n = 0, len(self._launches)
        while i < n:
            fused = self._fused.get(i)
            if fused is not None:
                fused.launch()
                i += fused.count
                continue
            launch, tensors, words = self._launches[i]
            launch(tensors, words)
            i += 1

    @property
    def launches_per_call(self) -> int:
        """Kernel-launching units a call runs (recorded steps less those fused away)."""
        return len(self._launches) - sum(f.count - f.launches for f in self._fused.values())

    @property
    def launches_per_replay(self) -> int:
        """Kernel launches one replay of the captured version makes: its steps' and, where the draw
        does not end the step itself, the tail's (carried values, re-derived words)."""
        if not self.capture:
            return self.launches_per_call
        if self._tail_in_draw:
            return self.launches_per_call
        tail = len(self.carry_copies) + (1 if self.n_tail else (2 if self.n_exprs > self.n_derived else 0))
        return self.launches_per_call + tail

    def _derive(self) -> None:
        from .. import kernels

        if self.n_derived:
            kernels.eval_words(self.words, self.expr_table, self.n_derived)

    def _carry_on_device(self) -> None:
        """token <- drawn, position <- position + 1: the values the next replay starts from."""
        from .. import kernels

        for slot, h in self.carry_copies:
            kernels.copy_rows(self._tensor(h).view(-1)[:1], self.words[slot : slot + 1], rows=1, row_elems=1,
                              src_rows=1, dst_rows=1)
        if self._tail_in_draw:
            return
        if self.n_tail:
            kernels.eval_words(self.words, self.expr_table[EXPR_WORDS * self.n_derived :], self.n_tail)
        elif self.n_exprs > self.n_derived:
            kernels.eval_words(self.words, self.expr_table[EXPR_WORDS * self.n_derived :], self.n_exprs - self.n_derived)
            self._derive()

    def _capture(self) -> None:
        import torch

        # Values any step can run on, so the warm-up launches touch valid rows.
        safe = {v.name: (v.default if v.default is not None else 0) for v in self.recording.values}
        self._write_words(self.recording.check_values(safe))
        stream = torch.cuda.Stream()
        stream.wait_stream(torch.cuda.current_stream())
        graphs = {}
        with torch.cuda.stream(stream):
            # Steps with a cheaper form within a limit are captured both ways; a call or a replay
            # takes the bounded graph while the values the host follows stay within every limit.
            for bounded in ((False, True) if self._bounds else (False,)):
                self._context["bounded"] = bounded
                self._derive()
                self._run_steps()
                stream.synchronize()
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph, stream=stream):
                    # The host wrote every word, derived ones included, before the first replay; each
                    # replay re-derives them for the next as it carries.
                    self._run_steps()
                    self._carry_on_device()
                stream.synchronize()
                graphs[bounded] = graph
            self._context["bounded"] = False
        torch.cuda.current_stream().wait_stream(stream)
        self._graph, self._graph_bounded = graphs[False], graphs.get(True)
        self._host_values = None   # the warm-up's values start no run of replays

    # -- calling -------------------------------------------------------------
    def _write_words(self, full: Mapping[str, int]) -> None:
        import torch

        # The words travel from one pinned buffer by an asynchronous copy: the last call's copy may
        # still be queued behind earlier work, and must have read the buffer before it is refilled.
        copied = vars(self).get("_words_copied")
        if copied is not None:
            copied.synchronize()
        self._host_values = {k: int(v) for k, v in full.items() if k != "__const__"}
        # Filled through the pinned tensor's numpy view in one assignment: word by word through
        # torch indexing this was a third of a millisecond a call, more than any launch of the chunk.
        filled = np.zeros(WORD_SLOTS, np.int64)
        for name, slot in self.slots.items():
            filled[slot] = int(full[name])
        for expr, slot in self.exprs.items():
            filled[slot] = expr.evaluate(full)
        self._host_words_np[:] = filled   # wraps to int32 as the device's own arithmetic does
        self.words.copy_(self.host_words, non_blocking=True)
        self._words_copied = torch.cuda.Event()
        self._words_copied.record()

    def _within_bounds(self, values: Mapping[str, int]) -> bool:
        """Whether every step with a bounded form stays within its limit at these per-call values."""
        at = {**values, "__const__": 0}
        return all(expr.evaluate(at) <= limit for expr, limit in self._bounds)

    def _replay_at(self, values: Mapping[str, int]) -> None:
        """One replay of the captured step from ``values`` (already on the device): the bounded
        graph where one was captured and the values allow it."""
        if self._graph_bounded is not None and self._within_bounds(values):
            self._graph_bounded.replay()
        else:
            self._graph.replay()

    def _after(self, values: Mapping[str, int], steps: int) -> dict[str, int]:
        """The per-call values ``steps`` runs after ``values``, as far as the host can follow them:
        what the body carries by a formula (``position + 1``); a value the device computes (the drawn
        token) keeps its last known number."""
        carry = self.recording.carry or {}
        values = dict(values)
        for _ in range(steps):
            at = {**values, "__const__": 0}
            for k, v in carry.items():
                if isinstance(v, Affine):
                    values[k] = v.evaluate(at)
                elif not isinstance(v, Handle):
                    values[k] = int(v)
        return values

    def write(self, resident: Resident, array) -> None:
        """Write a state or weight of the graph from a host array."""
        self.load()
        off = self.arena.resident_offsets[id(resident)]
        self.arena.view(off, resident.shape, resident.dtype).copy_(_host_tensor(np.asarray(array), resident.dtype))

    def read(self, resident: Resident) -> np.ndarray:
        """A state or weight as the device left it: a host copy, which ``push`` sends back."""
        self.load()
        off = self.arena.resident_offsets[id(resident)]
        array = from_torch(self.arena.view(off, resident.shape, resident.dtype))
        vars(self).setdefault("_read", {})[id(resident)] = array
        return array

    def push(self, resident: Resident) -> None:
        """Send to the device what the host wrote into the array ``read(resident)`` last returned
        (iron/common/graph/compiled.py:850-854: there the array is the buffer's own host memory)."""
        array = vars(self).get("_read", {}).get(id(resident))
        if array is None:
            raise ValueError("push() sends what read() returned: read the tensor first")
        self.write(resident, array)

    def upload(self, release=None, piece_bytes=None) -> None:
        """Copy every weight the versions hold into the arena, once an arena (``load`` does it too;
        the reference's keywords pace its host copies and mean nothing here)."""
        self.arena.load()

    def __call__(self, *tensors, **values):
        """Run the version: inputs are host arrays (or device tensors), values per-call ints.

        Returns the outputs (``DeviceOutput``) and, if the body carries values, the ``Carry`` last.
        """
        import torch

        rec = self.recording
        if len(tensors) != len(rec.inputs):
            raise TypeError(f"{rec.name}: takes {len(rec.inputs)} input tensor(s) "
                            f"{[h.buffer.name for h in rec.inputs]}, got {len(tensors)}")
        staged = []
        for h, t in zip(rec.inputs, tensors):
            shape = tuple(t.shape)
            if shape != h.shape:
                raise ValueError(f"{rec.name}: {h.buffer.name} takes {h.shape}, got {shape}")
            if isinstance(t, torch.Tensor):
                want = torch.bfloat16 if h.dtype is bfloat16 else getattr(torch, np.dtype(h.dtype).name)
                if t.dtype != want:
                    raise TypeError(f"{rec.name}: {h.buffer.name} takes {want}, got {t.dtype}")
                staged.append(t)
            else:
                a = np.asarray(t)
                if h.dtype is not bfloat16 and a.dtype != np.dtype(h.dtype):
                    raise TypeError(f"{rec.name}: {h.buffer.name} takes {np.dtype(h.dtype)}, got {a.dtype}")
                staged.append(_host_tensor(a, h.dtype))
        defaults = {v.name: v.default for v in rec.values if v.default is not None}
        full = rec.check_values({**defaults, **values})  # refused before any dispatch
        self.load()
        for i, (dst, src) in enumerate(zip(self.input_tensors, staged)):
            if src.device.type == "cpu" and not src.is_pinned():
                # A host array goes through a pinned buffer of this input's own (pageable memory would
                # make the copy a synchronous two-step one); the buffer is not refilled before the
                # last call's copy out of it has been made.
                held = self._staging.get(i)
                if held is None:
                    held = self._staging[i] = [torch.empty(dst.shape, dtype=dst.dtype).pin_memory(), None]
                if held[1] is not None:
                    held[1].synchronize()
                held[0].copy_(src.reshape(dst.shape))
                dst.copy_(held[0], non_blocking=True)
                held[1] = torch.cuda.Event()
                held[1].record()
            else:
                dst.copy_(src.reshape(dst.shape), non_blocking=True)
        self._write_words(full)
        if self._graph is not None:
            self._replay_at(full)
        else:
            if self.check:
                self._run_checked(full)
            else:
                self._run_steps()
        outs = []
        for h, t in zip(rec.outputs, self.output_tensors):
            rows = h.valid[0].evaluate(full) if 0 in h.valid else None
            outs.append(DeviceOutput(t, rows))
        if rec.carry is None:
            return outs[0] if len(outs) == 1 else tuple(outs)
        carried = Carry()
        for k, v in rec.carry.items():
            if isinstance(v, Handle):
                carried[k] = int(self._tensor(v).view(-1)[0].item())
            elif isinstance(v, Affine):
                carried[k] = v.evaluate(full)
            else:
                carried[k] = int(v)
        return (*outs, carried)

    @property
    def captured(self) -> bool:
        return self.capture

    def start(self, **values) -> None:
        """Run the version once from the given per-call values without reading anything back:
        the first of a run of device-carried steps (``replay`` runs the rest)."""
        rec = self.recording
        if rec.inputs:
            raise TypeError(f"{rec.name}: a version that takes tensors is called, not started")
        defaults = {v.name: v.default for v in rec.values if v.default is not None}
        full = rec.check_values({**defaults, **values})
        self.load()
        self._write_words(full)
        if self._graph is None:
            raise RuntimeError(f"{rec.name}: this version is not captured in a HIP graph")
        self._replay_at(full)

    def replay(self, n: int = 1) -> None:
        """Replay the captured step ``n`` more times, each starting from the values the last one carried."""
        if self._graph is None:
            raise RuntimeError(f"{self.recording.name}: this version is not captured in a HIP graph")
        if n <= 0:
            return
        known = vars(self).get("_host_values")
        if known is None:
            raise RuntimeError(f"{self.recording.name}: start() or a call runs the first step of a replayed run")
        # Every step's values are checked before any is launched, as a call's are: past a limit the
        # device would drop its cache writes and go on from stale rows without a word.  The carried
        # formulas move one way, so the first and the last replay bound the rest.
        first = self._after(known, 1)
        last = self._after(first, n - 1)
        try:
            self.recording.check_values(first)
            self.recording.check_values(last)
        except IndexError as e:
            raise IndexError(f"{e}; {n} replay(s) from {known} leave the limits") from None
        if self._graph_bounded is None:
            for _ in range(n):
                self._graph.replay()
        else:
            at = known
            for _ in range(n):
                at = self._after(at, 1)
                self._replay_at(at)
        self._host_values = last

    def _run_checked(self, full) -> None:
        """Per-step eager launches, each judged against its operator's ``reference()``."""
        import torch

        for step, (launch, tensors, words) in zip(self.recording.steps, self._launches):
            op = step.op
            plain = not any(h.index is not None or h.ids is not None or 0 in h.valid
                            for h in (*step.inputs.values(), *step.outputs.values()))
            ins = {n: from_torch(tensors[n]).reshape(h.shape) for n, h in step.inputs.items()} if plain else None
            launch(tensors, words)
            torch.cuda.current_stream().synchronize()
            tol = op.tolerance()
            if not plain or tol is None:
                continue
            declared = {b.name for b in op.outputs}  # scratch memory is written and not judged
            written = {n: from_torch(tensors[n]).reshape(h.shape) for n, h in step.outputs.items() if n in declared}
            values = {k: e.evaluate(full) for k, e in step.values.items()}
            extents = {k: v for k, v in values.items()
                       if next(m for m in op.declaration.per_calls if m.name == k).bounds is not None}
            others = {k: v for k, v in values.items() if k not in extents}
            at = op._at_extents(**extents) if extents else op
            verdicts = at.judge(ins, written, tol, at._call_reference(ins, values=others))
            bad = {n: v.detail for n, v in verdicts.items() if not v}
            if bad:
                raise AssertionError(f"{self.recording.name}: step {op.name}: {bad}")

    def release(self) -> None:
        self._graph = self._graph_bounded = None
        self._launches = []
        self._loaded_generation = None


class CarriedLoop:
    """A graph's carried values looped on the device (iron/common/graph/carried.py:189-276).

    ``first`` runs once from the host (a prompt chunk, or ``body`` itself); ``body`` -- a version
    that takes no tensor, captured in a HIP graph -- then runs as replays, each starting from the
    values the last run carried on the device, so the host only launches.  ``depth`` is the
    reference's count of runs in flight; a stream orders the replays here and it changes nothing.

    Raises:
        ValueError: ``first`` and ``body`` are not versions of one graph (one arena), ``body`` takes
            a tensor or carries nothing, or ``depth`` is under 1.
    """

    def __init__(self, first: CompiledGraph, body: CompiledGraph, depth: int = 2):
        if first.arena is not body.arena:
            raise ValueError("first and body are versions of one graph")
        if body.recording.inputs:
            raise ValueError(f"{body.recording.name}: the looped version takes no tensor, got "
                             f"{[h.buffer.name for h in body.recording.inputs]}")
        for version in (first, body):
            if not version.recording.carry:
                raise ValueError(f"{version.recording.name}: a version with carried values loops; this one carries none")
        if depth < 1:
            raise ValueError(f"depth is at least 1, got {depth}")
        self.first, self.body, self.depth = first, body, depth
        self._started = False

    def run(self, steps: int, /, *tensors, **values):
        """``start`` now, then ``steps``, each index yielded once launched."""
        self.start(*tensors, **values)
        return self.steps(steps)

    def start(self, *tensors, **values) -> None:
        """Run ``first`` on ``tensors`` and ``values``; what it carries is where ``body`` starts."""
        self.body.load()
        if not self.body.captured:
            raise RuntimeError(f"{self.body.recording.name}: the looped version is captured in a HIP graph (capture=True)")
        *_, carry = self.first(*tensors, **values)
        self._carry, self._started = dict(carry), True

    def steps(self, steps: int):
        """Run ``steps`` steps of ``body``, yielding each index once its replay is launched; what the
        steps wrote is read (``body.read``) after the last, which waits for them."""
        if not self._started:
            raise RuntimeError("start() runs the first version before the steps")
        for k in range(steps):
            if self._carry is not None:
                self.body.start(**self._carry)   # the first step takes first's carried values from the host
                self._carry = None
            else:
                self.body.replay(1)
            yield k

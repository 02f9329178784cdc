"""The operator declaration layer: ``param`` / ``tunable`` / ``per_call``, ``In`` / ``Out``,
``Select`` and the ``Operator`` base class.

The reference builds this on mlir-aie's ``aie.utils.compile.jit`` declaration DSL
(iron/common/declare/operator.py:84-637; semantics exercised by
iron/tests/common/test_declare.py).  Here it is self-contained: a subclass body is
the declaration, the constructor is keyword-only, tunables left ``None`` are open
until ``resolved()``, and ``build()`` returns a launch plan onto the C ABI instead
of an AIE array.  The AIE-only tunables (column counts, tile sizes, ...) are kept so
callers and profiles can pass them; they do not change the HIP launch.
"""

from __future__ import annotations

import copy
import dataclasses
import inspect
import math
from collections.abc import Callable, Mapping
from contextvars import ContextVar
from enum import Enum
from typing import Any, ClassVar

import numpy as np

from ..bf16 import bfloat16, itemsize
from .verify import Tolerance, Verdict, compare

_MISSING = object()

# The recorder of the graph body being run, if any (set by graph.Recorder).
graph_recorder: ContextVar[Any] = ContextVar("graph_recorder", default=None)

# name -> callable(op, *inputs, **kw): the CPU references, registered by the test oracle.
# The product never fills this: without a provider ``reference()`` raises.
REFERENCES: dict[str, Callable[..., Any]] = {}


class Unresolvable(Exception):
    """A tunable cannot be resolved (no value fits, or none was given and none is derivable)."""


class Precision(str, Enum):
    """The roundings a matmul may make beyond its reference's (iron/common/declare/precision.py:9).

    On the MFMA path every level computes alike: f32 partial sums, one rounding.
    """

    HIGHEST = "highest"
    HIGH = "high"
    MEDIUM = "medium"

    def __str__(self) -> str:
        return self.value


# ------------------------------------------------------------------ fields


class _Member:
    name: str = ""

    def __set_name__(self, owner, name):
        self.name = name


class Field(_Member):
    """A ``param()`` or ``tunable()``: read on the class it is the declaration, on an instance its value."""

    def __init__(self, *, kind, default=_MISSING, derive=None, array=False, repr=True, init=True,
                 domain=None):
        self.kind, self.default, self.derive = kind, default, derive
        self.array, self.repr, self.init, self.domain = array, repr, init, domain

    @property
    def tunable(self) -> bool:
        return self.kind == "tunable"

    def __get__(self, obj, cls):
        if obj is None:
            return self
        values = vars(obj)
        v = values.get(self.name)
        if v is None and (self.derive is not None or _is_factory(self.default)):
            # Computed from the other fields on first read; a field read while it is
            # being computed (a cycle) reads as None.
            busy = values.setdefault("_computing", set())
            if self.name in busy:
                return None
            busy.add(self.name)
            try:
                v = (self.derive or self.default)(obj)
            finally:
                busy.discard(self.name)
            if v is not None:
                values[self.name] = v
        return v


def _field_set(self, obj, value):
    vars(obj)[self.name] = value


# A data descriptor: reads go through __get__ even though the value lives in the instance dict.
Field.__set__ = _field_set


def _is_factory(default) -> bool:
    return callable(default) and not isinstance(default, (type, Enum))


def param(*, default=_MISSING, derive=None, array=False, repr=True, init=True) -> Any:
    """A construction field: a shape dimension or a compile-time constant."""
    return Field(kind="param", default=default, derive=derive, array=array, repr=repr, init=init)


def tunable(*, default=None, domain=None, repr=True, init=True) -> Any:
    """A choice about how to run; ``None`` is open until ``resolved()``."""
    return Field(kind="tunable", default=default, domain=domain, repr=repr, init=init)


class PerCall(_Member):
    """An int32 word the kernel reads each call: an extent (``bounds=``) or derived (``derive=``)."""

    def __init__(self, bounds=None, derive=None):
        self.bounds, self.derive = bounds, derive

    def __get__(self, obj, cls):
        if obj is None:
            return self
        extents = vars(obj).get("_extents", {})
        if self.name in extents:
            return extents[self.name]
        if self.derive is not None:
            return self.derive(obj)
        if self.bounds is not None:
            return _value_of(obj, self.bounds)
        return None


def per_call(*, bounds=None, derive=None) -> Any:
    return PerCall(bounds, derive)


class Select:
    """One of two shapes by a bool param (gemm.py:197-209)."""

    def __init__(self, flag, when_true, when_false):
        self.flag, self.when_true, self.when_false = flag, when_true, when_false


class OperandDecl(_Member):
    def __init__(self, dims, *, fills, drains, dtype=bfloat16, obj_shape=None, per=None, depth=None,
                 replicate=False, when=None, like=None, scratch=False, kept=False):
        self.dims, self.fills, self.drains, self.scratch, self.kept = dims, fills, drains, scratch, kept
        self.dtype, self.obj_shape, self.per, self.depth = dtype, obj_shape, per, depth
        self.replicate, self.when, self.like = replicate, when, like

    def __get__(self, obj, cls):
        if obj is None:
            return self
        return obj._operand(self)


def In(*dims, **kw) -> Any:  # noqa: N802 -- the reference's spelling
    return OperandDecl(dims, fills=True, drains=False, **kw)


def Out(*dims, **kw) -> Any:  # noqa: N802
    return OperandDecl(dims, fills=False, drains=True, **kw)


def InOut(*dims, **kw) -> Any:  # noqa: N802
    return OperandDecl(dims, fills=True, drains=True, **kw)


def Scratch(*dims, **kw) -> Any:  # noqa: N802
    """Device memory a kernel needs beside its operands (partial results): a graph places it
    in the arena as a transient; a call outside a graph allocates it once.  ``kept=True``: memory
    whose contents the kernel counts on finding as it left them (zero at first), which a graph
    places among its residents instead, one per step."""
    return OperandDecl(dims, fills=False, drains=False, scratch=True, **kw)


@dataclasses.dataclass(frozen=True)
class Operand:
    """A declared buffer of a constructed operator."""

    name: str
    shape: tuple[int, ...]
    dtype: Any
    fills: bool
    drains: bool
    replicate: bool = False
    kept: bool = False

    @property
    def host_shape(self) -> tuple[int, ...]:
        return self.shape

    @property
    def host_dtype(self):
        return np.float32 if self.dtype is bfloat16 else self.dtype

    @property
    def elements(self) -> int:
        return math.prod(self.shape)

    @property
    def nbytes(self) -> int:
        return self.elements * itemsize(self.dtype)


def _value_of(op, x):
    """A declaration-time reference (field, per-call, number) as its value on ``op``."""
    if isinstance(x, (Field, PerCall)):
        return getattr(op, x.name)
    return x


@dataclasses.dataclass
class Declaration:
    params: dict[str, Field]
    operands: list[OperandDecl]
    per_calls: list[PerCall]

    @property
    def tunables(self) -> dict[str, Field]:
        return {n: f for n, f in self.params.items() if f.tunable}

    @property
    def members(self) -> list[str]:
        return [*self.params, *(o.name for o in self.operands), *(p.name for p in self.per_calls)]


@dataclasses.dataclass(frozen=True)
class Built:
    """What ``build()`` made: the C-ABI entry point and a launch over device tensors.

    ``launch(tensors, words)``: ``tensors`` by operand name (torch CUDA tensors),
    ``words`` by per-call name (1-element int32 device tensors, or absent).
    """

    kernel: str
    launch: Callable[[Mapping[str, Any], Mapping[str, Any]], None]
    # ``(per-call value, limit)``: while that value stays within the limit, ``launch`` has a cheaper
    # form, which it takes when ``words["__context__"]["bounded"]`` is true.  The caller vouches for
    # the limit only as far as speed goes: the bounded form is correct for any value.
    bounded: tuple[str, int] | None = None


class Operator:
    """An operator, whose subclass body is its declaration.

    ``Op(**kw)`` constructs; ``Op.step(*handles, **kw)`` records a step inside a
    graph's body; ``op(*device_tensors)`` runs it alone, one tensor per declared
    buffer, inputs then outputs in declaration order.
    """

    declaration: ClassVar[Declaration] = Declaration({}, [], [])
    test: ClassVar[Any] = None
    reference_only: ClassVar[bool] = False
    dev: Any = None
    bound_values: dict[str, Any] = {}
    pinned: frozenset[str] = frozenset()

    def __init_subclass__(cls, **kwargs):
        super().__init_subclass__(**kwargs)
        params: dict[str, Field] = {}
        operands: dict[str, OperandDecl] = {}
        per_calls: dict[str, PerCall] = {}
        for klass in reversed(cls.__mro__):
            for name, member in vars(klass).items():
                for kind, table in ((Field, params), (OperandDecl, operands), (PerCall, per_calls)):
                    if isinstance(member, kind):
                        # A redeclared member takes its place in the redeclaring body.
                        table.pop(name, None)
                        table[name] = member
        cls.declaration = Declaration(params, list(operands.values()), list(per_calls.values()))

    # -- construction ------------------------------------------------------
    def __init__(self, *, bound_values=None, pinned=None, **given):
        decl = self.declaration
        unknown = [k for k in given if k not in decl.params]
        if unknown:
            raise TypeError(f"{type(self).__name__} has no parameter {unknown}")
        for n in given:
            f = decl.params[n]
            if f.derive is not None and given[n] is not None:
                raise TypeError(f"{type(self).__name__}.{n} is derived; it takes no value")
        if bound_values:
            self.bound_values = dict(bound_values)
        values = vars(self)
        for n, f in decl.params.items():
            values[n] = given[n] if given.get(n) is not None else None
        for n, f in decl.params.items():
            if values[n] is None and f.derive is None and not _is_factory(f.default):
                if f.default is _MISSING:
                    if not f.tunable:
                        raise TypeError(f"{type(self).__name__} needs {n}=")
                else:
                    values[n] = f.default
        for n in decl.params:  # factories and derivations, in dependency order by lazy reads
            getattr(self, n)
        if pinned is None:
            pinned = frozenset(n for n in decl.tunables if given.get(n) is not None)
        self.pinned = pinned
        self.validate()
        self._check_complete()

    def _check_complete(self) -> None:
        if not any(f.tunable and vars(self)[n] is None and f.init for n, f in self.declaration.params.items()):
            self.compatible()

    def validate(self) -> None:
        """Refuse what no tunable could mend; runs at construction."""

    def compatible(self) -> None:
        """Refuse what the chosen tunables cannot run; runs once every tunable is known."""

    def resolve(self, dev):
        """Return a copy with every open tunable filled."""
        return self

    def resolved(self, dev=None):
        return self.resolve(dev if dev is not None else self.dev)

    def replace(self, **changes):
        bound_values = changes.pop("bound_values", self.bound_values)
        pinned = changes.pop("pinned", self.pinned)
        decl = self.declaration
        given = {n: vars(self)[n] for n, f in decl.params.items() if f.derive is None}
        given.update(changes)
        return type(self)(bound_values=bound_values, pinned=pinned, **given)

    def copy(self):
        return copy.copy(self)

    # -- declared members --------------------------------------------------
    def _dims(self, dims) -> tuple[int, ...]:
        if len(dims) == 1 and isinstance(dims[0], Select):
            s = dims[0]
            dims = s.when_true if _value_of(self, s.flag) else s.when_false
        out = []
        for d in dims:
            v = _value_of(self, d)
            if isinstance(v, (tuple, list)):
                out.extend(int(x) for x in v)
            elif v is not None:  # a None dimension is omitted (test_declare.py:112-124)
                out.append(int(v))
        return tuple(out)

    def _operand(self, decl: OperandDecl) -> Operand | None:
        if decl.when is not None and not _value_of(self, decl.when):
            return None
        src = decl if decl.like is None else decl.like
        dtype = _value_of(self, src.dtype)
        return Operand(decl.name, self._dims(src.dims), dtype, decl.fills, decl.drains, decl.replicate, decl.kept)

    @property
    def buffers(self) -> list[Operand]:
        found = (self._operand(d) for d in self.declaration.operands if not d.scratch)
        return [b for b in found if b is not None]

    @property
    def scratch(self) -> list[Operand]:
        found = (self._operand(d) for d in self.declaration.operands if d.scratch)
        return [b for b in found if b is not None]

    @property
    def inputs(self) -> list[Operand]:
        return [b for b in self.buffers if b.fills]

    @property
    def outputs(self) -> list[Operand]:
        return [b for b in self.buffers if b.drains]

    @property
    def bound_extents(self) -> dict[str, Any]:
        return {m.name: self.bound_values[m.name] for m in self.declaration.per_calls
                if m.bounds is not None and m.name in self.bound_values}

    def _at_extents(self, **extents):
        """A copy whose extents read as the given numbers (a bounded call's)."""
        at = copy.copy(self)
        vars(at)["_extents"] = {**vars(self).get("_extents", {}), **extents}
        return at

    # -- graph recording hooks ------------------------------------------------
    def _leading_field(self, decl: OperandDecl):
        """The declared field an operand's first (present) dimension is, if it is one."""
        src = decl if decl.like is None else decl.like
        dims = src.dims
        if len(dims) == 1 and isinstance(dims[0], Select):
            s = dims[0]
            dims = s.when_true if _value_of(self, s.flag) else s.when_false
        for d in dims:
            if _value_of(self, d) is not None:
                return d if isinstance(d, Field) else None
        return None

    def bind_views(self, inputs: Mapping[str, Any], outputs) -> dict[str, Any]:
        """The per-call extents a call's handles bind: ``x[:n]`` on an operand whose first
        dimension an extent bounds binds that extent to ``n`` (record.py:886-904)."""
        bound = {}
        for m in self.declaration.per_calls:
            if m.bounds is None:
                continue
            for decl in self.declaration.operands:
                h = inputs.get(decl.name)
                if h is None or 0 not in getattr(h, "valid", {}):
                    continue
                if self._leading_field(decl) is m.bounds:
                    bound.setdefault(m.name, h.valid[0])
        return bound

    def output_valid(self, name: str, inputs: Mapping[str, Any]) -> dict[int, Any]:
        """The bound an output inherits: that of the extent bounding its first dimension."""
        decl = next(d for d in self.declaration.operands if d.name == name)
        lead = self._leading_field(decl)
        for m in self.declaration.per_calls:
            if m.bounds is not None and m.bounds is lead and self.bound_values.get(m.name) is not None:
                return {0: self.bound_values[m.name]}
        return {}

    def output_shape(self, name: str, inputs: Mapping[str, Any]):
        """The shape a graph sees the output in, where it is not the declared one (an
        elementwise result keeps its input's shape); None for the declared shape."""
        return None

    def takes_view(self, name: str) -> bool:
        """Whether operand ``name`` may be a per-call view (an index, a window, a gather)."""
        return False

    def use_value(self, name: str, bound_to=None) -> None:
        if not any(m.name == name for m in self.declaration.per_calls):
            raise TypeError(f"{type(self).__name__} declares no per-call value {name!r}")
        self.bound_values = {**self.bound_values, name: bound_to}

    @property
    def name(self) -> str:
        shown = [f"{n}_{_spelled(vars(self)[n])}" for n, f in self.declaration.params.items()
                 if f.repr and vars(self)[n] is not None]
        return "_".join([type(self).__name__, *shown])

    def __repr__(self) -> str:
        return self.name

    def design_key(self):
        own = tuple((n, _spelled(vars(self)[n])) for n in self.declaration.params)
        if self.bound_values:
            names = {k: None if v is None else getattr(v, "name", str(v)) for k, v in self.bound_values.items()}
            own += (("values", tuple(sorted(names.items()))),)
        return type(self), own

    # -- what an operator computes ------------------------------------------
    def build(self) -> Built:
        raise NotImplementedError(f"{type(self).__name__}.build() is not implemented")

    def tolerance(self) -> Tolerance | None:
        return None

    def ops(self) -> int:
        return sum(b.elements for b in self.outputs)

    def reference(self, *inputs, **kwargs):
        """The CPU reference of this operator: supplied by the test oracle, never by the product."""
        for klass in type(self).__mro__:
            fn = REFERENCES.get(klass.__name__)
            if fn is not None:
                return fn(self, *inputs, **kwargs)
        raise NotImplementedError(
            f"{type(self).__name__}.reference(): no CPU reference is registered; the oracle is test "
            "infrastructure (import oracle; oracle.install())"
        )

    def _call_reference(self, inputs: Mapping[str, Any], outputs: Mapping[str, Any] | None = None,
                        values: Mapping[str, Any] | None = None) -> dict[str, Any]:
        name = type(self).__name__
        declared = [b.name for b in self.inputs]
        if sorted(inputs) != sorted(declared):
            raise ValueError(f"{name} takes the inputs {declared}, not {sorted(inputs)}")
        required = [d.name for d in self.declaration.operands if d.fills and d.when is None]
        optional = {d.name: inputs[d.name] for d in self.declaration.operands
                    if d.fills and d.when is not None and d.name in inputs}
        extra = {k: v for k, v in (values or {}).items() if v is not None}
        result = self.reference(*(inputs[n] for n in required), **optional, **extra)
        results = result if isinstance(result, tuple) else (result,)
        written = [b.name for b in self.outputs]
        if len(results) != len(written) or any(r is None for r in results):
            raise ValueError(f"{name}.reference returned {len(results)} results for {written}")
        return dict(zip(written, results))

    def judge(self, inputs, written, tolerance: Tolerance, expected=None) -> dict[str, Verdict]:
        if expected is None:
            expected = self._call_reference(inputs)
        names = [b.name for b in self.outputs]
        for given, what in ((written, "written"), (expected, "expected")):
            if sorted(given) != sorted(names):
                raise ValueError(f"{type(self).__name__} writes {names}; the {what} buffers are {sorted(given)}")
        bound = None
        if tolerance.kind == "bound":
            bound = tolerance.bound(*(inputs[b.name] for b in self.inputs))
        return {n: compare(np.reshape(written[n], np.shape(expected[n])), expected[n], tolerance, bound=bound)
                for n in names}

    # -- calling -----------------------------------------------------------
    @classmethod
    def call_operands(cls, args, kwargs):
        """Split a call into inputs by name, outputs and other keywords (operator.py:240-260)."""
        ins = [d for d in cls.declaration.operands if d.fills]
        required = [d.name for d in ins if d.when is None]
        optional = {d.name for d in ins if d.when is not None}
        given = {k: v for k, v in kwargs.items() if k in optional and v is not None}
        if len(args) < len(required):
            raise TypeError(f"{cls.__name__} takes {len(required)} positional operand(s) "
                            f"({', '.join(required)}), got {len(args)}")
        bound = {**dict(zip(required, args)), **given}
        inputs = {d.name: bound[d.name] for d in ins if d.name in bound}
        rest = {k: v for k, v in kwargs.items() if k not in optional}
        return inputs, list(args[len(required):]), rest

    @classmethod
    def infer(cls, input_shapes: Mapping[str, tuple[int, ...]], **kw) -> dict[str, Any]:
        """Shape params from operand shapes (overridden where a declaration cannot say)."""
        raise NotImplementedError(f"{cls.__name__}.infer() is not implemented")

    @classmethod
    def step(cls, *operands, **kwargs):
        """Record a step inside a graph's body: ``GEMV.step(w, h, **kw)``."""
        recorder = graph_recorder.get()
        if recorder is None:
            raise TypeError(f"{cls.__name__}.step() is for a graph's body")
        return recorder.call(cls, operands, kwargs)

    def compile(self) -> Built:
        built = vars(self).get("_built")
        if built is None:
            if self.reference_only:
                raise TypeError(f"{type(self).__name__} is reference-only: it never compiles")
            built = vars(self)["_built"] = self.resolved().build()
        return built

    def __call__(self, *args, **kwargs):
        if (recorder := graph_recorder.get()) is not None:
            return recorder.call(self, args, kwargs)
        import torch

        names = [b.name for b in self.buffers]
        if len(args) != len(names) or not all(isinstance(a, torch.Tensor) for a in args):
            raise TypeError(
                f"{type(self).__name__} runs outside a graph's body on device tensors, one per "
                f"declared buffer {names}; got {[type(a).__name__ for a in args]}"
            )
        for b, t in zip(self.buffers, args):
            if t.numel() != b.elements:
                raise ValueError(f"{type(self).__name__}: {b.name} takes {b.shape}, got {tuple(t.shape)}")
        words = {k: v for k, v in kwargs.items() if v is not None}
        unknown = [k for k in words if not any(m.name == k for m in self.declaration.per_calls)]
        if unknown:
            raise TypeError(f"{type(self).__name__} declares no per-call value {unknown}")
        self.compile().launch(dict(zip(names, args)), words)
        torch.cuda.current_stream().synchronize()
        return args[len(self.inputs):] if len(self.outputs) != 1 else args[-1]


def _spelled(v) -> str:
    if isinstance(v, bool):
        return str(int(v))
    if isinstance(v, float):
        return repr(v).replace(".", "p").replace("-", "n").replace("+", "")
    if isinstance(v, (list, tuple)):
        return "x".join(str(x) for x in v)
    if isinstance(v, Enum):
        return str(v.value)
    if isinstance(v, type):
        return v.__name__
    return f"{v}"


def ceildiv(a: int, b: int) -> int:
    return -(-a // b)


def signature_names(fn) -> list[str]:
    return list(inspect.signature(fn).parameters)

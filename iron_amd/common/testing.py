"""Checking one operator on the GPU against its CPU reference, and timing it.

The names are the reference's (iron/common/testing.py:33-297: ``Case``, ``Testing``, ``vectors``,
``run_test``, ``time_call``) so an operator's declared cases and a test that runs them read the same.
Here the device is an MI355X, buffers are torch tensors in HBM, and a latency is the time between
two HIP events recorded on the launching stream.
"""

from __future__ import annotations

import dataclasses
import logging
from collections.abc import Callable, Iterable, Mapping
from typing import Any

import numpy as np

from ..bf16 import bfloat16, from_torch, round_bf16, to_torch
from .verify import Tolerance, Verdict

__all__ = ["Case", "Testing", "Vectors", "run_test", "time_call", "vectors"]

log = logging.getLogger(__name__)


@dataclasses.dataclass(frozen=True)
class Case:
    """Constructor keywords for one instance of an operator, and which suites pick it up:
    ``extensive`` (the long run only), ``bench`` (also timed), ``lower`` (built but not run)."""

    kwargs: dict = dataclasses.field(default_factory=dict)
    extensive: bool = False
    id: str | None = None
    bench: bool = False
    lower: bool = False

    @property
    def label(self) -> str:
        if self.id:
            return self.id
        return "-".join(f"{key}_{value}" for key, value in self.kwargs.items())


@dataclasses.dataclass(frozen=True)
class Testing:
    """What an operator class declares for its tests: ``cases`` -- ``Case`` objects and/or callables
    ``(cls, device) -> cases`` for sizes that depend on the device -- and optionally ``draw``, which
    maps a built operator to keyword arguments for ``vectors`` when random inputs will not do."""

    __test__ = False          # not a pytest class, despite the name

    cases: Any
    draw: Callable[[Any], dict[str, Any]] | None = None

    def resolve(self, cls: type, dev=None) -> list[Case]:
        entries = (self.cases,) if callable(self.cases) else tuple(self.cases)
        flat: list[Case] = []
        for entry in entries:
            flat.extend(entry(cls, dev) if callable(entry) else (entry,))
        return flat


@dataclasses.dataclass
class Vectors:
    """Inputs and expected outputs by buffer name; indexing looks in both."""

    inputs: dict[str, np.ndarray]
    outputs: dict[str, np.ndarray]

    def __getitem__(self, name: str) -> np.ndarray:
        source = self.inputs if name in self.inputs else self.outputs
        return source[name]


def _is_integer(dtype) -> bool:
    return dtype is not bfloat16 and np.dtype(dtype).kind not in "fc"


def vectors(op, *, seed: int = 42, scale: float = 4.0, normal: Iterable = (), centered: Iterable = (),
            given: Mapping | None = None) -> Vectors:
    """Seeded inputs for every input buffer of ``op`` (in declaration order, so a seed fixes them),
    with the outputs its ``reference()`` computes from them (iron/common/testing.py:95-144).

    Floats are uniform on ``[0, scale)``; operands listed in ``normal`` are ``N(0, 1) * scale``;
    those in ``centered`` are shifted down by ``scale / 2``.  Integers are uniform on
    ``[0, scale]``.  ``given`` maps an operand either to a ready array or to a shape to draw at.

    Raises:
        ValueError: ``normal`` / ``centered`` / ``given`` names an operand that is not an input.
    """
    supplied = {operand.name: value for operand, value in (given or {}).items()}
    gaussian = {operand.name for operand in normal}
    shifted = {operand.name for operand in centered}
    strangers = (set(supplied) | gaussian | shifted) - {b.name for b in op.inputs}
    if strangers:
        raise ValueError(f"{type(op).__name__} has no input {sorted(strangers)}")
    rng = np.random.default_rng(seed)
    drawn: dict[str, np.ndarray] = {}
    for buffer in op.inputs:
        hint = supplied.get(buffer.name)
        if isinstance(hint, np.ndarray):
            drawn[buffer.name] = hint
            continue
        shape = tuple(hint) if hint is not None else buffer.host_shape
        if _is_integer(buffer.dtype):
            drawn[buffer.name] = rng.integers(0, int(scale) + 1, shape).astype(buffer.dtype)
            continue
        sample = rng.standard_normal(shape) if buffer.name in gaussian else rng.random(shape)
        values = (sample * scale).astype(np.float32)
        if buffer.name in shifted:
            values = values - np.float32(scale / 2)
        drawn[buffer.name] = round_bf16(values) if buffer.dtype is bfloat16 else values.astype(buffer.dtype)
    return Vectors(drawn, op._call_reference(drawn))


def _torch_dtype(dtype):
    import torch

    return torch.bfloat16 if dtype is bfloat16 else getattr(torch, np.dtype(dtype).name)


def _upload(buffer, array):
    import torch

    if buffer.dtype is bfloat16:
        return to_torch(array).cuda()
    return torch.from_numpy(np.ascontiguousarray(array, dtype=buffer.dtype)).cuda()


def time_call(fn: Callable, *args, bytes_moved: int = 0, ops: float = 0.0, warmup: int = 2, iters: int = 20,
              record: Callable[[str, float], object] | None = None, **kwargs) -> float:
    """Median latency of ``fn(*args, **kwargs)`` in microseconds over ``iters`` runs, each bracketed
    by a pair of HIP events on the current stream, after ``warmup`` untimed runs.  With ``record``
    (e.g. pytest's ``record_property``) also reports the median absolute deviation and, given
    ``bytes_moved`` / ``ops``, GB/s and GOP/s."""
    import torch

    for _ in range(warmup):
        fn(*args, **kwargs)
    samples = np.empty(iters, dtype=np.float64)
    for i in range(iters):
        begin = torch.cuda.Event(enable_timing=True)
        end = torch.cuda.Event(enable_timing=True)
        begin.record()
        fn(*args, **kwargs)
        end.record()
        end.synchronize()
        samples[i] = begin.elapsed_time(end) * 1e3      # ms -> us
    latency = float(np.median(samples))
    spread = float(np.median(np.abs(samples - latency)))
    if record is not None:
        seconds = latency * 1e-6
        record("Latency", latency)
        record("Latency MAD", spread)
        if bytes_moved:
            record("Bandwidth", bytes_moved / seconds / 1e9)
        if ops:
            record("Throughput", ops / seconds / 1e9)
    log.info("Latency (us): %.1f ± %.1f", latency, spread)
    return latency


def run_test(operator, inputs, outputs=None, *, tolerance: Tolerance, timed_iters: int = 20,
             record: Callable[[str, float], object] | None = None) -> dict[str, Verdict]:
    """Run ``operator`` once on the GPU from ``inputs`` (a ``Vectors`` or a dict by buffer name),
    judge each output buffer against ``outputs`` (default: the reference's) under ``tolerance``,
    then time the bare launch.  Returns the failing outputs' verdicts by name -- empty means pass.

    Raises:
        TypeError: ``operator`` is not a declared ``Operator``.
        ValueError: ``inputs`` does not name exactly the operator's input buffers.
    """
    import torch

    from .declare import Operator

    if isinstance(inputs, Vectors):
        outputs = inputs.outputs if outputs is None else outputs
        inputs = inputs.inputs
    if not isinstance(operator, Operator):
        raise TypeError(f"run_test runs one declared Operator, not {operator!r}")
    expected_names = [b.name for b in operator.inputs]
    if sorted(inputs) != sorted(expected_names):
        raise ValueError(f"{type(operator).__name__} takes the inputs {expected_names}, not {sorted(inputs)}")
    built = operator.compile()
    device_buffers, moved = {}, 0
    for buffer in operator.buffers:
        if buffer.fills:
            device_buffers[buffer.name] = _upload(buffer, inputs[buffer.name])
        else:
            device_buffers[buffer.name] = torch.zeros(buffer.host_shape, dtype=_torch_dtype(buffer.dtype), device="cuda")
        moved += buffer.nbytes
    operator(*device_buffers.values())
    results = {b.name: from_torch(device_buffers[b.name]) for b in operator.buffers if b.drains}
    verdicts = operator.judge(inputs, results, tolerance, outputs)
    failed = {name: verdict for name, verdict in verdicts.items() if not verdict}
    for name, verdict in failed.items():
        log.warning("%s: %s", name, verdict.detail)
    time_call(lambda: built.launch(device_buffers, {}), bytes_moved=moved, ops=operator.resolved().ops(),
              iters=timed_iters, record=record)
    return failed

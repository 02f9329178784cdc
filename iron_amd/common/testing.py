"""How an operator is checked against its reference on the device, and timed.

``Case`` / ``Testing`` / ``vectors`` / ``run_test`` / ``time_call`` as in
iron/common/testing.py:33-297; the device is the MI355X and time is taken with HIP
events around replays of the launch on the current stream.
"""

from __future__ import annotations

import logging
from collections.abc import Callable, Iterable, Mapping
from dataclasses import dataclass, field
from typing import Any

import numpy as np

from ..bf16 import bfloat16, from_torch, round_bf16, to_torch
from .verify import Tolerance, Verdict

logger = logging.getLogger(__name__)

__all__ = ["Case", "Testing", "Vectors", "run_test", "time_call", "vectors"]


@dataclass(frozen=True)
class Case:
    """One construction of an operator (the constructor's keywords and how the suites use it)."""

    kwargs: dict = field(default_factory=dict)
    extensive: bool = False
    id: str | None = None
    bench: bool = False
    lower: bool = False

    @property
    def label(self) -> str:
        return self.id or "-".join(f"{k}_{v}" for k, v in self.kwargs.items())


@dataclass(frozen=True)
class Testing:
    """An operator's cases and, where inputs have preconditions, how to draw them."""

    __test__ = False

    cases: Any
    draw: Callable[[Any], dict[str, Any]] | None = None

    def resolve(self, cls: type, dev=None) -> list[Case]:
        out = []
        for c in [self.cases] if callable(self.cases) else self.cases:
            out += list(c(cls, dev)) if callable(c) else [c]
        return out


@dataclass
class Vectors:
    inputs: dict[str, np.ndarray]
    outputs: dict[str, np.ndarray]

    def __getitem__(self, name: str) -> np.ndarray:
        return self.inputs[name] if name in self.inputs else self.outputs[name]


def vectors(op, *, seed: int = 42, scale: float = 4.0, normal: Iterable = (), centered: Iterable = (),
            given: Mapping | None = None) -> Vectors:
    """Random inputs for ``op``'s declared buffers and ``op.reference()``'s outputs (testing.py:95-144).

    Uniform on ``[0, scale)`` by default, ``N(0,1) * scale`` for the operands in ``normal``.
    """
    given_names = {o.name: v for o, v in (given or {}).items()}
    normal_names = {o.name for o in normal}
    centered_names = {o.name for o in centered}
    unknown = (given_names.keys() | normal_names | centered_names) - {b.name for b in op.inputs}
    if unknown:
        raise ValueError(f"{type(op).__name__} has no input {sorted(unknown)}")
    rng = np.random.default_rng(seed)
    inputs = {}
    for b in op.inputs:
        value = given_names.get(b.name)
        if isinstance(value, np.ndarray):
            inputs[b.name] = value
            continue
        shape = b.host_shape if value is None else tuple(value)
        if b.dtype is not bfloat16 and np.dtype(b.dtype).kind not in "fc":
            t = rng.integers(0, int(scale) + 1, shape).astype(b.dtype)
        else:
            draw = rng.standard_normal if b.name in normal_names else rng.random
            t = (draw(shape) * scale).astype(np.float32)
            if b.name in centered_names:
                t = t - np.float32(scale / 2)
            t = round_bf16(t) if b.dtype is bfloat16 else t.astype(b.dtype)
        inputs[b.name] = t
    return Vectors(inputs, op._call_reference(inputs))


def _to_device(b, array):
    import torch

    if b.dtype is bfloat16:
        return to_torch(array).cuda()
    return torch.from_numpy(np.ascontiguousarray(array, dtype=b.dtype)).cuda()


def _empty_device(b):
    import torch

    dtype = torch.bfloat16 if b.dtype is bfloat16 else getattr(torch, np.dtype(b.dtype).name)
    return torch.zeros(b.host_shape, dtype=dtype, device="cuda")


def time_call(fn: Callable, *args, bytes_moved: int = 0, ops: float = 0.0, warmup: int = 2, iters: int = 20,
              record: Callable[[str, float], object] | None = None, **kwargs) -> float:
    """Median device latency (µs) of ``iters`` runs of ``fn(*args)``, each between two HIP events."""
    import torch

    for _ in range(warmup):
        fn(*args, **kwargs)
    times = []
    for _ in range(iters):
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        fn(*args, **kwargs)
        stop.record()
        stop.synchronize()
        times.append(start.elapsed_time(stop) * 1e3)
    latency = float(np.median(times))
    mad = float(np.median(np.abs(np.asarray(times) - latency)))
    if record is not None:
        record("Latency", latency)
        record("Latency MAD", mad)
        if bytes_moved:
            record("Bandwidth", bytes_moved / (latency * 1e-6) / 1e9)
        if ops:
            record("Throughput", ops / (latency * 1e-6) / 1e9)
    logger.info("Latency (us): %.1f ± %.1f", latency, mad)
    return latency


def run_test(operator, inputs, outputs=None, *, tolerance: Tolerance, timed_iters: int = 20,
             record: Callable[[str, float], object] | None = None) -> dict[str, Verdict]:
    """Build ``operator``, run it on the GPU, judge every output against its reference, time it.

    Returns each failing output's ``Verdict`` by name; empty where all passed.
    """
    from .declare import Operator

    if isinstance(inputs, Vectors):
        inputs, outputs = inputs.inputs, inputs.outputs
    if not isinstance(operator, Operator):
        raise TypeError(f"run_test runs one declared Operator, not {operator!r}")
    declared = [b.name for b in operator.inputs]
    if sorted(inputs) != sorted(declared):
        raise ValueError(f"{type(operator).__name__} takes the inputs {declared}, not {sorted(inputs)}")
    operator.compile()
    args, produced, total_bytes = [], {}, 0
    for b in operator.buffers:
        buf = _to_device(b, inputs[b.name]) if b.fills else _empty_device(b)
        if b.drains:
            produced[b.name] = buf
        args.append(buf)
        total_bytes += b.nbytes
    operator(*args)
    written = {name: from_torch(buf) for name, buf in produced.items()}
    verdicts = operator.judge(inputs, written, tolerance, outputs)
    errors = {name: v for name, v in verdicts.items() if not v}
    for name, v in errors.items():
        logger.warning("%s: %s", name, v.detail)
    launch = operator.compile().launch
    named = dict(zip([b.name for b in operator.buffers], args))
    time_call(lambda: launch(named, {}), bytes_moved=total_bytes, ops=operator.resolved().ops(),
              iters=timed_iters, record=record)
    return errors

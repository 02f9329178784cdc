"""``Tolerance`` and ``compare``: how an output is judged against its reference.

The reference takes these from mlir-aie (``aie.utils.verify``); their admitted
intervals are restated by iron/tests/support/judging.py:35-84 and exercised by
iron/tests/common/test_judging.py:75-174, which this follows:

  exact     equal after rounding to the output dtype
  relative  |got - want| < rtol * (|got| + |want|), floor atol
  ulps      within n bf16 steps (or atol)
  bound     |got - want| <= fn(*inputs)
NaN fails; ``max_mismatch_frac`` of the elements may miss; ``range_frac`` also
admits an error of that share of the reference's largest magnitude.
"""

from __future__ import annotations

import dataclasses
from collections.abc import Callable
from typing import Any

import numpy as np

from ..bf16 import round_bf16, to_bits


@dataclasses.dataclass(frozen=True)
class Tolerance:
    kind: str = "relative"
    rtol: float | None = None
    atol: float | None = None
    ulps: int | None = None
    bound: Callable[..., Any] | None = None
    max_mismatch_frac: float = 0.0
    range_frac: float | None = None
    note: str = ""

    def __init__(self, rtol=None, atol=None, max_mismatch_frac=0.0, note="", *, kind="relative",
                 ulps=None, bound=None, range_frac=None):
        object.__setattr__(self, "kind", kind)
        object.__setattr__(self, "rtol", rtol)
        object.__setattr__(self, "atol", atol)
        object.__setattr__(self, "ulps", ulps)
        object.__setattr__(self, "bound", bound)
        object.__setattr__(self, "max_mismatch_frac", max_mismatch_frac)
        object.__setattr__(self, "range_frac", range_frac)
        object.__setattr__(self, "note", note)

    @classmethod
    def exact(cls, note: str = "") -> "Tolerance":
        return cls(kind="exact", note=note)

    @classmethod
    def relative(cls, rtol: float, atol: float | None = None, range_frac: float | None = None,
                 note: str = "") -> "Tolerance":
        return cls(rtol=rtol, atol=atol, range_frac=range_frac, note=note)

    @classmethod
    def bf16_ulps(cls, n: int, atol: float | None = None, note: str = "") -> "Tolerance":
        return cls(kind="ulps", ulps=n, atol=atol, note=note)

    @classmethod
    def bounded(cls, fn: Callable[..., Any], note: str = "") -> "Tolerance":
        return cls(kind="bound", bound=fn, note=note)


@dataclasses.dataclass(frozen=True)
class Verdict:
    ok: bool
    n_mismatch: int
    n_checked: int
    max_abs_err: float
    detail: str = ""

    def __bool__(self) -> bool:
        return self.ok


def _bf16_ordinal(x: np.ndarray) -> np.ndarray:
    """bf16 values on a line of integers, adjacent values one apart."""
    bits = to_bits(x).astype(np.int32)
    return np.where(bits & 0x8000, -(bits & 0x7FFF), bits)


def compare(got, want, tol: Tolerance, bound=None) -> Verdict:
    """Judge ``got`` against ``want`` by ``tol``; truthy on pass."""
    got = np.asarray(got)
    want = np.asarray(want)
    if got.shape != want.shape:
        got = got.reshape(want.shape)
    integer = np.issubdtype(want.dtype, np.integer)
    g = got.astype(np.float64)
    w = want.astype(np.float64)
    err = np.abs(g - w)
    if tol.kind == "exact":
        bad = got != want if integer else ~((g == w) | (np.isnan(g) & np.isnan(w)))
    elif tol.kind == "bound":
        if bound is None:
            raise ValueError("a bound tolerance is judged with its bound evaluated on the inputs")
        bad = ~(err <= np.broadcast_to(np.asarray(bound, np.float64).reshape(w.shape), w.shape))
    elif tol.kind == "ulps":
        steps = np.abs(_bf16_ordinal(round_bf16(g)) - _bf16_ordinal(round_bf16(w)))
        bad = steps > (tol.ulps or 0)
        if tol.atol is not None:
            bad &= ~(err < tol.atol)
    else:
        r = tol.rtol or 0.0
        floor = float(np.finfo(np.float32).tiny) if tol.atol is None else tol.atol
        bad = ~((err < r * (np.abs(g) + np.abs(w))) | (err < floor) | (g == w))
    if tol.range_frac is not None and tol.kind in ("relative", "ulps"):
        finite = np.isfinite(w)
        scale = float(np.max(np.abs(w), where=finite, initial=0.0))
        bad &= ~(err <= tol.range_frac * scale)
    # Equal infinities pass; NaN anywhere fails.
    bad = np.where(np.isinf(w) & (g == w), False, bad)
    bad |= np.isnan(g) & ~(np.isnan(w) & (tol.kind == "exact"))
    n_bad, n = int(np.count_nonzero(bad)), int(bad.size)
    finite_err = err[np.isfinite(err)]
    max_err = float(finite_err.max()) if finite_err.size else 0.0
    ok = n_bad <= tol.max_mismatch_frac * n
    detail = ""
    if n_bad:
        i = int(np.argmax(np.where(bad, np.nan_to_num(err, nan=np.inf, posinf=np.inf), -1).reshape(-1)))
        detail = (
            f"{n_bad}/{n} elements outside the tolerance ({tol.kind}); worst at flat index {i}: "
            f"got {g.reshape(-1)[i]!r}, want {w.reshape(-1)[i]!r}; max |err| {max_err:.6g}"
        )
    return Verdict(ok, n_bad, n, max_err, detail)

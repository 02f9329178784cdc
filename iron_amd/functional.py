"""Functions for a graph's body, under ``torch.nn.functional``'s names (iron/functional.py:30-129).

Each records the operator steps that compute it and returns their handle.  Weights are a
checkpoint's ``(out, in)``, as ``torch.nn.Linear`` stores them.
"""

from __future__ import annotations

import math

from .common.declare import Precision
from .operators.gemm import GEMM
from .operators.gemv import GEMV
from .operators.rms_norm import RMSNorm
from .operators.rope import RoPE
from .operators.silu import SiLU

BF16_EPS = 2.0**-7  # bfloat16's machine epsilon


def linear(x, weight, bias=None, *, precision: Precision = Precision.HIGHEST, **gemv):
    """Return ``x @ weight.T``, plus ``bias`` on every row if given.

    One row runs on GEMV, which always rounds once in float32; several rows run on the MFMA
    GEMM reading the weight as stored (``b_col_maj``) -- at every ``precision`` the same
    kernel: f32 partial sums, one rounding (the reference's flm.ProjectionGEMM at
    MEDIUM/HIGH has no counterpart here).

    Raises:
        ValueError: ``x`` of another rank, or GEMV tunables for several rows.
    """
    if len(x.shape) not in (1, 2):
        raise ValueError(f"linear(): x {tuple(x.shape)} is not (in,) or (rows, in)")
    one_row = len(x.shape) == 1 or x.shape[0] == 1
    if one_row:
        y = GEMV.step(weight, x, **gemv)
    elif gemv:
        raise ValueError(f"linear(): {x.shape[0]} rows take no GEMV {sorted(gemv)}")
    else:
        y = GEMM.step(x, weight, b_col_maj=True, precision=precision)
    if bias is None:
        return y
    # A row added to every row, also for GEMV's one-dimensional output.
    rows = math.prod(y.shape) // bias.shape[0]
    return (y.reshape(rows, bias.shape[0]) + bias).reshape(y.shape)


def _last_axis(name: str, x, normalized_shape) -> None:
    given = (normalized_shape,) if isinstance(normalized_shape, int) else tuple(normalized_shape)
    if given != tuple(x.shape[-1:]):
        raise ValueError(f"{name}(): normalized_shape {list(given)} is not the last axis of input "
                         f"{list(x.shape)}; only ({x.shape[-1]},) is normalized")


def rms_norm(x, normalized_shape, weight=None, eps: float | None = None):
    """``x`` over the RMS of its last axis, times ``weight`` if given; ``eps`` None is bf16's epsilon."""
    _last_axis("rms_norm", x, normalized_shape)
    if eps is None:
        eps = BF16_EPS
    return RMSNorm.step(x, weight=weight, epsilon=eps)


def silu(x):
    """Apply SiLU, ``x * sigmoid(x)``, as torch's."""
    return SiLU.step(x)


def rope(x, angles):
    """``x`` ``(rows, head_dim)`` turned by RoPE, a row of ``angles`` per row."""
    return RoPE.step(x, angles)

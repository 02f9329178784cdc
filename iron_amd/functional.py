"""``torch.nn.functional``-style recorders for a graph's body (the reference's iron/functional.py:30-129).

Calling one of these inside a body appends the operator step(s) that compute it and hands back the
result's handle.  Matrices are ``(out_features, in_features)``, the way ``torch.nn.Linear`` and every
checkpoint store them, so both GEMV and GEMM read a weight row as one contiguous run of K.
"""

from __future__ import annotations

import math

from .common.declare import Precision
from .operators.gemm import GEMM
from .operators.gemv import GEMV
from .operators.rms_norm import RMSNorm
from .operators.rope import RoPE
from .operators.silu import SiLU

BF16_EPS = 2.0**-7   # machine epsilon of bfloat16 (8 significand bits), the default norm epsilon


def linear(x, weight, bias=None, *, precision: Precision = Precision.HIGHEST, **gemv):
    """``x @ weight.T (+ bias)``.

    Dispatch by row count: a single row (``(in,)`` or ``(1, in)``) records the bandwidth-bound
    ``GEMV``, anything taller the MFMA ``GEMM`` with ``b_col_maj`` (the weight as stored).  Both
    accumulate in float32 and round once whatever ``precision`` says: the reference's reduced-precision
    projection kernels have no equivalent here, the field is only carried.  ``gemv`` passes tunables
    to the single-row case.

    Raises:
        ValueError: ``x`` is neither a vector nor a matrix; or GEMV tunables came with several rows.
    """
    rank = len(x.shape)
    if rank not in (1, 2):
        raise ValueError(f"linear(): x {tuple(x.shape)} is not (in,) or (rows, in)")
    rows = 1 if rank == 1 else x.shape[0]
    if rows > 1 and gemv:
        raise ValueError(f"linear(): {rows} rows take no GEMV {sorted(gemv)}")
    if rows == 1:
        product = GEMV.step(weight, x, **gemv)
    else:
        product = GEMM.step(x, weight, b_col_maj=True, precision=precision)
    if bias is None:
        return product
    # Broadcast the bias over rows; a GEMV's flat output is viewed as one row for the purpose.
    width = bias.shape[0]
    as_rows = product.reshape(math.prod(product.shape) // width, width)
    return (as_rows + bias).reshape(product.shape)


def rms_norm(x, normalized_shape, weight=None, eps: float | None = None):
    """RMS normalisation over the last axis (``normalized_shape`` must name exactly that axis),
    scaled by ``weight`` when given.  ``eps=None`` means bfloat16's machine epsilon, as torch picks
    the dtype's.

    Raises:
        ValueError: ``normalized_shape`` is not ``x``'s last axis.
    """
    wanted = (normalized_shape,) if isinstance(normalized_shape, int) else tuple(normalized_shape)
    last = tuple(x.shape[-1:])
    if wanted != last:
        raise ValueError(f"rms_norm(): normalized_shape {list(wanted)} is not the last axis of input "
                         f"{list(x.shape)}; only ({x.shape[-1]},) is normalized")
    return RMSNorm.step(x, weight=weight, epsilon=BF16_EPS if eps is None else eps)


def silu(x):
    """``x * sigmoid(x)`` elementwise."""
    return SiLU.step(x)


def rope(x, angles):
    """Rotate the rows of ``x`` (``(rows, head_dim)``, two-halves convention) by ``angles``, whose
    rows are spread evenly over ``x``'s."""
    return RoPE.step(x, angles)

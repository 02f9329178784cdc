"""bfloat16 on the host without a numpy bf16 dtype.

A host array of a bf16 operand is a ``float32`` numpy array whose every
value is exactly representable in bfloat16 (a "bf16-valued" array).
``round_bf16`` rounds any float32 array onto that set, to nearest even, as
``astype(ml_dtypes.bfloat16)`` does in the reference; ``to_bits`` /
``from_bits`` give the 16-bit storage the device holds.
"""

from __future__ import annotations

import numpy as np


class bfloat16:  # noqa: N801 -- spelled as the dtype it stands for
    """Marker for a bf16 operand's element type (2 bytes on the device)."""

    itemsize = 2
    name = "bfloat16"

    def __new__(cls, *a, **k):
        raise TypeError("bfloat16 is a dtype marker; use round_bf16() for values")


def itemsize(dtype) -> int:
    """Bytes one element of ``dtype`` takes on the device."""
    if dtype is bfloat16:
        return 2
    return np.dtype(dtype).itemsize


def round_bf16(x) -> np.ndarray:
    """Return ``x`` (any float array) as float32 rounded to the nearest bf16, ties to even."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32)
    bias = ((u >> np.uint32(16)) & np.uint32(1)) + np.uint32(0x7FFF)
    r = (u + bias) & np.uint32(0xFFFF0000)
    # NaN stays NaN (quiet), whatever its payload.
    nan = (u & np.uint32(0x7FFFFFFF)) > np.uint32(0x7F800000)
    r = np.where(nan, u | np.uint32(0x00400000), r).astype(np.uint32)
    return r.view(np.float32).reshape(x.shape)


def is_bf16_valued(x) -> bool:
    x = np.ascontiguousarray(x, dtype=np.float32)
    return not bool((x.view(np.uint32) & np.uint32(0xFFFF)).any())


def to_bits(x) -> np.ndarray:
    """The uint16 storage of ``round_bf16(x)``."""
    r = round_bf16(x)
    return (r.view(np.uint32) >> np.uint32(16)).astype(np.uint16).reshape(r.shape)


def from_bits(bits) -> np.ndarray:
    """bf16 storage (uint16) as a bf16-valued float32 array."""
    bits = np.ascontiguousarray(bits, dtype=np.uint16)
    return (bits.astype(np.uint32) << np.uint32(16)).view(np.float32).reshape(bits.shape)


def to_torch(x, device=None):
    """A bf16-valued (or any float) numpy array as a torch.bfloat16 tensor."""
    import torch

    t = torch.from_numpy(to_bits(x).view(np.int16)).view(torch.bfloat16)
    return t if device is None else t.to(device)


def from_torch(t) -> np.ndarray:
    """A torch.bfloat16 tensor (any device) as a bf16-valued float32 numpy array."""
    import torch

    if t.dtype != torch.bfloat16:
        return t.detach().cpu().numpy()
    return from_bits(t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16))

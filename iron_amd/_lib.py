"""ctypes binding of ``libiron_hip.so`` (the C ABI declared in ``include/iron_hip.h``).

There is no fallback: if the library is missing or a symbol is absent, loading
raises, and every operator call goes through here.
"""

from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_float, c_int, c_int64, c_void_p
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "libiron_hip.so"

_P = c_void_p

# name -> (restype, argtypes); one entry per declaration of include/iron_hip.h.
SIGNATURES = {
    "iron_version": (c_int, []),
    "iron_last_error": (c_char_p, []),
    "iron_gemm_bf16": (c_int, [_P, _P, _P, c_int, c_int, c_int, c_int, c_int, _P, _P, _P]),
    "iron_gemv_bf16": (c_int, [_P, _P, _P, c_int, c_int, c_int, c_int, _P, _P]),
    "iron_gemv_bf16_tuned": (c_int, [_P, _P, _P, c_int, c_int, c_int, c_int, _P, c_int, c_int, _P]),
    "iron_gemm_residual_bf16": (c_int, [_P, _P, _P, _P, c_int, c_int, c_int, c_float, _P, _P]),
    "iron_gemm_residual_norm_workspace_bytes": (c_int64, [c_int, c_int, c_int]),
    "iron_gemm_residual_norm_bf16": (c_int, [_P, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_float, c_float, _P, _P, _P]),
    "iron_gemm_gated_bf16": (c_int, [_P, _P, _P, _P, c_int, c_int, c_int, c_int, _P, _P]),
    "iron_gemv_fused_bf16": (c_int, [_P, _P, _P, _P, c_float, _P, c_float, _P, c_int, c_int, c_int, _P]),
    "iron_decode_qkv_bf16": (
        c_int,
        [_P, _P, c_float, _P, _P, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, _P, _P, c_int, _P],
    ),
    "iron_decode_heads_bf16": (
        c_int,
        [_P, _P, _P, _P, _P, c_int, c_float, _P, _P, c_int, c_int, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, _P],
    ),
    "iron_decode_qkv_embed_bf16": (
        c_int,
        [_P, _P, c_int, _P, _P, c_float, _P, _P, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, _P, _P, c_int, _P],
    ),
    "iron_gemm_gated_pair_bf16": (c_int, [_P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, _P, _P]),
    "iron_prefill_qkv_bf16": (c_int, [_P] * 8 + [c_int] * 5 + [_P, _P]),
    "iron_prefill_qkv_cache_bf16": (c_int, [_P] * 8 + [c_int] * 6 + [_P, _P, _P]),
    "iron_rmsnorm_bf16": (c_int, [_P, _P, _P, c_int, c_int, c_float, _P, _P]),
    "iron_rmsnorm_add_bf16": (c_int, [_P, _P, _P, _P, c_int, c_int, c_float, _P, _P]),
    "iron_rope_bf16": (c_int, [_P, _P, _P, c_int, c_int, c_int, c_int, _P, _P]),
    "iron_rope_partial_bf16": (c_int, [_P, _P, _P, c_int, c_int, c_int, c_int, c_int, _P, _P]),
    "iron_silu_bf16": (c_int, [_P, _P, c_int64, _P, _P]),
    "iron_mul_bf16": (c_int, [_P, _P, _P, c_int64, _P, _P]),
    "iron_add_bf16": (c_int, [_P, _P, _P, c_int64, _P, _P]),
    "iron_row_broadcast_bf16": (c_int, [_P, _P, _P, c_int, c_int, c_int, _P, _P]),
    "iron_silu_mul_bf16": (c_int, [_P, _P, _P, c_int64, _P, _P]),
    "iron_mha_prefill_bf16": (
        c_int,
        [_P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_int,
         c_int, _P, _P, _P],
    ),
    "iron_mha_decode_bf16": (
        c_int,
        [_P, _P, _P, _P, c_int, c_int, c_int, c_int, c_float, c_int, c_int, _P, _P, _P],
    ),
    "iron_mha_decode_workspace_bytes": (c_int64, [c_int, c_int]),
    "iron_mha_decode_tuned_bf16": (
        c_int,
        [_P, _P, _P, _P, c_int, c_int, c_int, c_int, c_float, c_int, c_int, _P, _P, c_int, c_int, _P],
    ),
    "iron_mha_decode_static_bf16": (
        c_int,
        [_P, _P, _P, _P, c_int, c_int, c_int, c_int, c_float, c_int, c_int, _P, _P],
    ),
    "iron_mha_decode_static_max_bytes": (c_int64, []),
    "iron_mha_prefill_at_bf16": (
        c_int,
        [_P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_int, _P, _P, _P, c_int, _P],
    ),
    "iron_mha_decode_at_bf16": (
        c_int,
        [_P, _P, _P, _P, c_int, c_int, c_int, c_int, c_float, c_int, _P, _P, c_int, _P, _P],
    ),
    "iron_gather_rows": (c_int, [_P, _P, _P, c_int, c_int, c_int64, _P, _P]),
    "iron_copy_rows": (c_int, [_P, _P, c_int, c_int64, c_int64, c_int64, c_int, c_int, _P, _P, _P, _P]),
    "iron_argmax_bf16": (c_int, [_P, c_int, _P, _P, c_int, _P, _P, _P]),
    "iron_unary_bf16": (c_int, [_P, _P, c_int64, c_int, c_float, c_float, _P, _P]),
    "iron_axpy_bf16": (c_int, [_P, _P, _P, c_int64, c_float, _P, _P]),
    "iron_layernorm_bf16": (c_int, [_P, _P, _P, c_int, c_int, c_float, _P, _P]),
    "iron_softmax_bf16": (c_int, [_P, c_int, _P, _P, c_int, c_int, c_float, _P, _P]),
    "iron_sample_workspace_bytes": (c_int64, [c_int]),
    "iron_sample_bf16": (c_int, [_P, c_int, _P, c_int, _P, c_int, _P, _P, _P, c_int, _P, _P, _P]),
    "iron_sample_advance_bf16": (c_int, [_P, c_int, _P, c_int, _P, c_int, _P, _P, _P, c_int, _P, _P, _P, c_int, _P,
                                         c_int, _P]),
    "iron_eval_words": (c_int, [_P, c_int, _P, c_int, _P]),
}


class IronHipError(RuntimeError):
    """An entry point refused its arguments or its launch failed."""


_lib = None


def lib() -> ctypes.CDLL:
    """The loaded library, every symbol typed; raises if it was never built."""
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise IronHipError(
                f"{LIB_PATH} is missing: build it with `python -m iron_amd.build` "
                "(there is no CPU fallback)"
            )
        handle = ctypes.CDLL(str(LIB_PATH))
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(handle, name)  # AttributeError names a missing symbol
            fn.restype, fn.argtypes = restype, argtypes
        _lib = handle
    return _lib


def check(code: int, what: str) -> None:
    if code != 0:
        text = lib().iron_last_error().decode()
        kind = "refused" if code == 1 else f"failed (hipError {code})"
        raise IronHipError(f"{what} {kind}: {text}")


def ptr(t) -> int | None:
    """Device address of a torch tensor (None stays NULL)."""
    return None if t is None else t.data_ptr()


def current_stream() -> int:
    import torch

    return torch.cuda.current_stream().cuda_stream

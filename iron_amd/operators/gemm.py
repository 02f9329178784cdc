"""GEMM: ``C = A @ B`` on the bf16 MFMA matrix cores.

The reference's operator (iron/operators/gemm.py:143-735): ``b_col_maj`` reads B as
stored by a checkpoint, ``(N, K)``; ``c_col_maj`` writes ``(N, M)``; per-call ``valid``
bounds the rows and ``valid_k`` the reduction.  Every ``Precision`` runs the same kernel
(``iron_gemm_bf16``): f32 partial sums, one rounding -- ``HIGHEST``'s contract.
"""

from __future__ import annotations

from typing import Any

import numpy as np

from ..bf16 import bfloat16
from ..common.declare import Built, In, Operator, Out, Precision, Select, param, per_call, tunable
from ..common.testing import Case, Testing
from ..common.verify import Tolerance

# fmt: off
#   M,     K,     N, b_col_maj, c_col_maj   (gemm.py:40-62, tile columns dropped)
_REGULAR = [
    (2048, 2048, 2048, False, False), (2048, 2048, 2048, True, False), (2048, 2048, 2048, True, True),
    (384, 1536, 1792, True, False), (1792, 896, 1152, False, True), (896, 1792, 640, False, True),
    (192, 384, 64, True, True), (32, 1152, 2048, True, True),
]
_EXTENSIVE = [
    (2048, 2048, 8192, True, False), (2048, 8192, 2048, True, False), (2048, 64, 2048, True, False),
    (2048, 64, 8192, True, False), (1024, 2560, 10240, False, False), (2048, 2048, 512, True, False),
]
# fmt: on


def _cases(cls, dev=None):
    out = []
    for rows, extensive in ((_REGULAR, False), (_EXTENSIVE, True)):
        for M, K, N, b, c in rows:
            kwargs = dict(M=M, K=K, N=N, b_col_maj=b, c_col_maj=c, precision=Precision.HIGHEST)
            out.append(Case(kwargs, extensive=extensive, bench=(M, K, N) == (2048, 2048, 2048)))
    return out


class GEMM(Operator):
    """``C = A @ B`` on 16x16x32 bf16 MFMAs, float32 sums, one rounding: 256 x 256, 128 x 128 or 64 x 64
    tiles by the shape (and, under a per-call row bound, by the bound, chosen on the device)."""

    test = Testing(_cases, draw=lambda op: dict(normal=(op.A,)))

    M: int = param()
    K: int = param()
    N: int = param()
    # The reference's AIE tunables: accepted, carried, not used by the HIP launch.
    tile_m: int = tunable()
    tile_k: int = tunable(default=64)
    tile_n: int = tunable(default=64)
    num_aie_columns: int = tunable()
    placement: Any = tunable()
    b_col_maj: bool = param(default=False, array=True)
    c_col_maj: bool = param(default=False, array=True)
    precision: Precision = param(default=Precision.HIGHEST, array=True)
    accumulate_f32: bool = param(default=True, array=True)
    input_dtype: Any = param(default=bfloat16, repr=False)
    output_dtype: Any = param(default=bfloat16, repr=False)

    A = In(M, K, dtype=input_dtype)
    B = In(Select(b_col_maj, (N, K), (K, N)), dtype=input_dtype)
    C = Out(Select(c_col_maj, (N, M), (M, N)), dtype=output_dtype)
    valid = per_call(bounds=M)
    valid_k = per_call(bounds=K)

    def validate(self) -> None:
        if self.input_dtype is not bfloat16 or self.output_dtype is not bfloat16:
            raise ValueError("GEMM: the MFMA kernel is bf16 in, bf16 out")
        if self.K % 8:
            raise ValueError(f"GEMM: K ({self.K}) must be a multiple of 8: a lane loads 8 bf16 at a time")
        if not self.b_col_maj and self.N % 8:
            raise ValueError(f"GEMM: N ({self.N}) must be a multiple of 8 when B is (K, N)")

    @classmethod
    def infer(cls, shapes, b_col_maj=False, **kw):
        a, b = shapes["A"], shapes["B"]
        if len(a) != 2 or len(b) != 2:
            raise ValueError(f"A {a} and B {b} are matrices")
        k, n = (b[1], b[0]) if b_col_maj else (b[0], b[1])
        if k != a[1]:
            raise ValueError(f"A {a} and B {b} (b_col_maj={b_col_maj}) disagree on K")
        return dict(M=a[0], K=a[1], N=n)

    def ops(self) -> int:
        return 2 * self.M * self.K * self.N

    def tolerance(self) -> Tolerance:
        """C's one rounding: 2 units of 2^-8 of ``|A| @ |B|`` (4 at MEDIUM) (gemm.py:704-735)."""
        units = 4.0 if self.precision == Precision.MEDIUM else 2.0

        def bound(A, B):
            a = np.asarray(A, np.float32)
            b = np.asarray(B, np.float32)
            b = b.T if self.b_col_maj else b
            err = units * (np.abs(a) @ np.abs(b)) * 2.0**-8
            return err.T if self.c_col_maj else err

        return Tolerance.bounded(bound, note=f"{units:g} units of |A| @ |B|")

    def build(self) -> Built:
        from .. import kernels

        M, N, K, b, c = self.M, self.N, self.K, self.b_col_maj, self.c_col_maj

        def launch(t, words):
            kernels.gemm(t["A"], t["B"], t["C"], M=M, N=N, K=K, b_col_maj=b, c_col_maj=c,
                         valid=words.get("valid"), valid_k=words.get("valid_k"))

        return Built("iron_gemm_bf16", launch)

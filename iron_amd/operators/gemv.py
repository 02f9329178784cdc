"""GEMV: ``C = A @ B`` with A the ``(M, K)`` weight and B the ``(K,)`` activation.

The reference's operator (iron/operators/gemv.py:79-421) on the HBM-bound HIP kernel
``iron_gemv_bf16``: f32 accumulation, one rounding.  ``num_batches`` / ``repeat`` batch
it (grouped-query scores).  The AIE tunables are accepted and carried; the launch
shape is ``rows_per_wave`` x ``k_split`` (open = the kernel's heuristic).
"""

from __future__ import annotations

from ..common.declare import Built, In, Operator, Out, param, per_call, tunable
from ..common.testing import Case, Testing
from ..common.verify import Tolerance


def _cases(cls, dev=None):
    # M, K[, num_batches[, repeat]] -- the reference's shapes (gemv.py:24-76)
    plain = [(128, 128), (2048, 8192), (8192, 2048), (1536, 12288)]
    batched = [(256, 128, 4), (256, 128, 100), (448, 64, 192), (64, 1536, 8), (1026, 64, 2), (1024, 1024, 2),
               (512, 64, 32)]
    repeated = [(256, 128, 8, 4), (256, 128, 4, 4), (1024, 1024, 4, 2), (2048, 64, 32, 4)]
    # ... and Llama-3.2-1B's decode projections and head.
    llama = [(2048, 2048), (512, 2048), (8192, 2048), (128256, 2048)]
    out = [Case(dict(M=m, K=k), bench=m * k >= 2048 * 8192) for m, k in plain + llama]
    out += [Case(dict(M=m, K=k, num_batches=b)) for m, k, b in batched]
    out += [Case(dict(M=m, K=k, num_batches=b, repeat=r)) for m, k, b, r in repeated]
    return out


class GEMV(Operator):
    """``C = A @ B``, a row of A per wave (or several, or a slice of K)."""

    test = Testing(_cases, draw=lambda op: dict(normal=(op.A, op.B)))

    M: int = param()
    K: int = param()
    # None: a single batch, with no batch dimension.
    num_batches: int | None = param(default=None)
    # Batches per matrix of A (grouped-query scores): no repeated copy.
    repeat: int = param(default=1)
    num_matrices: int | None = param(
        derive=lambda op: None if op.num_batches is None else op.num_batches // op.repeat
    )
    # The reference's AIE tunables: accepted, carried, not used by the HIP launch.
    num_aie_columns: int = tunable()
    num_channels: int = tunable()
    tile_size_input: int = tunable()
    tile_size_output: int = tunable()
    kernel_vector_size: int = tunable(repr=False)
    # The HIP launch shape; open = chosen by the kernel from M, K and the batch count.
    rows_per_wave: int = tunable(domain=(1, 2, 4, 8), repr=False)
    k_split: int = tunable(domain=(1, 2, 4), repr=False)

    A = In(num_matrices, M, K)
    B = In(num_batches, K)
    C = Out(num_batches, M)
    valid = per_call(bounds=M)

    def validate(self):
        if self.repeat < 1 or (self.num_batches or 1) % self.repeat:
            raise ValueError(f"GEMV: repeat ({self.repeat}) must divide num_batches ({self.num_batches})")
        tso, tsi = self.tile_size_output, self.tile_size_input
        if tso is not None and tsi is not None and not (tso % tsi == 0 and tso >= tsi):
            raise ValueError(f"GEMV: tile_size_output ({tso}) must be a multiple of tile_size_input ({tsi})")
        if self.K % 8:
            raise ValueError(f"GEMV: K ({self.K}) must be a multiple of 8: a lane loads 8 bf16 at a time")

    @classmethod
    def infer(cls, shapes, **kw):
        a, b = shapes["A"], shapes["B"]
        if len(a) == 3:
            batches = 1
            for s in b[:-1]:
                batches *= s
            return dict(M=a[1], K=a[2], num_batches=batches, repeat=batches // a[0])
        if len(a) != 2:
            raise ValueError(f"A {a} is not (M, K) or (matrices, M, K)")
        return dict(M=a[0], K=a[1])

    def ops(self) -> int:
        return 2 * self.M * self.K * (self.num_batches or 1)

    def tolerance(self) -> Tolerance:
        """C accumulates in f32 and rounds once (gemv.py:419-421)."""
        return Tolerance.relative(0.04, 1e-3, note="f32 accumulation, rounded once")

    def build(self) -> Built:
        from .. import kernels

        M, K, batches, repeat = self.M, self.K, self.num_batches or 1, self.repeat
        rpw, ks = self.rows_per_wave or 0, self.k_split or 0

        def launch(t, words):
            kernels.gemv(t["A"], t["B"], t["C"], M=M, K=K, batches=batches, repeat=repeat,
                         valid=words.get("valid"), rows_per_wave=rpw, k_split=ks)

        return Built("iron_gemv_bf16", launch)

"""Every operator's declared cases on the GPU against its CPU reference
(iron/tests/operators/test_catalog.py:53-76): construct, draw ``vectors(op, seed=42)``,
dispatch, judge every output element by ``op.tolerance()``, and by the stated bf16
tolerance (rtol 1e-2 / atol 1e-2 where the values are O(1))."""

import numpy as np
import pytest

import oracle
from iron_amd.common.testing import run_test, vectors
from iron_amd.operators import CATALOG

pytestmark = pytest.mark.gpu
oracle.install()

CASES = [
    pytest.param(cls, case, id=f"{name}-{case.label}")
    for name, cls in CATALOG.items()
    for case in cls.test.resolve(cls, None)
    # The largest cases' CPU references take minutes (16 K-row attention in numpy).
    if not (name == "MHA" and case.kwargs.get("seq_len", 0) >= 16384)
]


@pytest.mark.parametrize("cls,case", CASES)
def test_operator_case(cuda, cls, case, record_property):
    op = cls(**case.kwargs)
    draw = cls.test.draw(op) if cls.test.draw else {}
    # Inputs of scale 4 overflow nothing but make attention one-hot; draw them at scale 1 there.
    scale = 1.0 if cls.__name__ == "MHA" else 4.0
    v = vectors(op, seed=42, scale=scale, **draw)
    errors = run_test(op, v, tolerance=op.tolerance(), timed_iters=3, record=record_property)
    assert not errors, {k: e.detail for k, e in errors.items()}


def test_operator_api_refusals(cuda):
    import torch

    from iron_amd.operators import GEMV, MHA, RoPE

    op = GEMV(M=64, K=64)
    with pytest.raises(TypeError, match="one per declared buffer"):
        op(torch.zeros(64, 64, device="cuda", dtype=torch.bfloat16))
    with pytest.raises(TypeError, match=r"step\(\) is for a graph's body"):
        GEMV.step(None, None)
    with pytest.raises(ValueError, match="must divide"):
        GEMV(M=64, K=64, num_batches=6, repeat=4)
    with pytest.raises(ValueError, match="multiple of"):
        MHA(num_heads=6, num_KV_heads=4, seq_len=64)
    with pytest.raises(ValueError, match="must divide rows"):
        RoPE(rows=12, cols=64, angle_rows=5)

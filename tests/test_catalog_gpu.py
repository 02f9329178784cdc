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


LONGEST = [
    pytest.param(case, id=f"MHA-{case.label}")
    for case in CATALOG["MHA"].test.resolve(CATALOG["MHA"], None)
    if case.kwargs.get("seq_len", 0) >= 16384
]


@pytest.mark.parametrize("case", LONGEST)
def test_longest_attention_cases_on_sampled_queries(cuda, case):
    """The catalog's 16384-row attention cases, whose whole reference takes the host minutes: the
    operator runs whole through its own call, and every head of a sample of queries (both ends, tile
    edges, random rows) is judged by the operator's tolerance against the one-query reference of that
    query over its keys -- the same operator at ``seq_len=1``, which the causal case is row by row."""
    import torch

    from iron_amd.bf16 import from_torch, to_torch
    from iron_amd.common.verify import compare

    cls = CATALOG["MHA"]
    op = cls(**case.kwargs)
    assert op.causal and not op.heads_interleaved and not op.kv_interleaved
    v = vectors(op, seed=42, scale=1.0)
    Q, Kc, Vc = (v.inputs[n] for n in ("Q", "K", "V"))
    O = torch.zeros(op.O.host_shape, dtype=torch.bfloat16, device="cuda")
    op(*(to_torch(a).cuda() for a in (Q, Kc, Vc)), O)
    got = from_torch(O)
    S = op.seq_len
    rng = np.random.default_rng(1)
    rows = sorted({0, 1, 63, 64, 127, 128, 8191, 8192, S - 129, S - 128, S - 1, *rng.integers(0, S, 9).tolist()})
    for r in rows:
        one = cls(num_heads=op.num_heads, num_KV_heads=op.num_KV_heads, seq_len=1, kv_len=r + 1, d=op.d)
        want = np.asarray(one.reference(Q[:, r : r + 1], Kc[:, : r + 1], Vc[:, : r + 1])).reshape(op.num_heads, op.d)
        verdict = compare(got[:, r], want, op.tolerance())
        assert verdict, f"query {r}: {verdict.detail}"
        assert np.all(np.abs(got[:, r] - want) <= 1e-2 + 1e-2 * np.abs(want)), f"query {r}"


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

"""Pin the CPU oracle (oracle/ops.py) before anything is judged by it.

Each check is independent of the oracle's own formula: a float64 library routine,
a row-by-row closed form, brute force on tiny inputs, or an invariant, chosen so
a dropped term, wrong sign/index or transposed operand fails.
"""

import math

import numpy as np
import pytest

from iron_amd.bf16 import from_bits, is_bf16_valued, round_bf16, to_bits
from oracle import ops


def bf(rng, *shape, scale=1.0):
    return round_bf16(rng.standard_normal(shape).astype(np.float32) * scale)


# ------------------------------------------------------------------ bf16 helper
def test_round_bf16_is_round_to_nearest_even():
    # 1 + 2^-8 is exactly between 1 and 1 + 2^-7: ties go to the even mantissa (1.0).
    x = np.array([1 + 2**-8, 1 + 2**-7 + 2**-8, 1 + 2**-8 + 2**-20, -1 - 2**-8], np.float32)
    want = np.array([1.0, 1 + 2**-6, 1 + 2**-7, -1.0], np.float32)
    assert np.array_equal(round_bf16(x), want)
    assert is_bf16_valued(round_bf16(x))
    assert np.array_equal(from_bits(to_bits(x)), round_bf16(x))


def test_round_bf16_matches_torch():
    torch = pytest.importorskip("torch")
    x = np.random.default_rng(0).standard_normal(1 << 16).astype(np.float32) * 37.0
    want = torch.from_numpy(x).to(torch.bfloat16).float().numpy()
    assert np.array_equal(round_bf16(x), want)


# ------------------------------------------------------------------------ GEMM
@pytest.mark.parametrize("b_col_maj", [False, True])
@pytest.mark.parametrize("c_col_maj", [False, True])
def test_gemm_against_float64(b_col_maj, c_col_maj):
    rng = np.random.default_rng(1)
    M, K, N = 48, 96, 40
    A, B = bf(rng, M, K), bf(rng, K, N)
    Bs = np.ascontiguousarray(B.T) if b_col_maj else B
    got = ops.gemm(A, Bs, b_col_maj=b_col_maj, c_col_maj=c_col_maj)
    exact = A.astype(np.float64) @ B.astype(np.float64)
    exact = exact.T if c_col_maj else exact
    assert got.shape == exact.shape
    # One rounding of an f32 sum: within one bf16 ulp of the float64 result.
    assert np.all(np.abs(got - exact) <= 2.0**-7 * np.abs(exact) + 1e-6)


def test_gemm_valid_k_ignores_what_lies_past_the_bound():
    rng = np.random.default_rng(2)
    A, B = bf(rng, 16, 64), bf(rng, 64, 24)
    poisoned_a, poisoned_b = A.copy(), B.copy()
    poisoned_a[:, 40:] = np.nan
    poisoned_b[40:] = np.nan
    got = ops.gemm(poisoned_a, poisoned_b, valid_k=40)
    assert np.array_equal(got, ops.gemm(A[:, :40], B[:40]))


def test_gemm_bound_is_two_units_of_abs_product():
    A = np.array([[1.0, -2.0]], np.float32)
    B = np.array([[3.0], [4.0]], np.float32)
    assert np.allclose(ops.gemm_bound(A, B), 2 * 11 * 2.0**-8)


# ------------------------------------------------------------------------ GEMV
def test_gemv_against_float64_and_batches():
    rng = np.random.default_rng(3)
    A, B = bf(rng, 24, 64), bf(rng, 64)
    exact = A.astype(np.float64) @ B.astype(np.float64)
    got = ops.gemv(A, B)
    assert np.all(np.abs(got - exact) <= 2.0**-7 * np.abs(exact) + 1e-6)
    # Batched with repeat: batch b uses matrix b // repeat.
    A3, B2 = bf(rng, 2, 8, 32), bf(rng, 4, 32)
    got = ops.gemv(A3, B2, repeat=2)
    for b in range(4):
        assert np.array_equal(got[b], ops.gemv(A3[b // 2], B2[b]))


# ------------------------------------------------------------------------ RoPE
def _block_major_expected(x, angles, rows, angle_rows):
    """Row r uses angle row r // (rows // angle_rows); written out row by row."""
    cols = x.shape[-1]
    half = cols // 2
    per = rows // angle_rows
    out = np.empty((rows, cols), dtype=np.float32)
    for r in range(rows):
        a = r // per
        cos = angles[a, 0::2].astype(np.float32)
        sin = angles[a, 1::2].astype(np.float32)
        x1, x2 = x[r, :half].astype(np.float32), x[r, half:].astype(np.float32)
        out[r, :half] = x1 * cos - x2 * sin
        out[r, half:] = x2 * cos + x1 * sin
    return round_bf16(out)


@pytest.mark.parametrize("rows,angle_rows", [(8, 2), (1024, 1), (4, 4), (13, 13), (12, 4)])
def test_rope_reference_convention(rows, angle_rows):
    """The shapes and the array_equal bar of the reference's own convention test."""
    rng = np.random.default_rng(0)
    cols, half = 32, 16
    x = round_bf16(rng.standard_normal((rows, cols)))
    angles = np.zeros((angle_rows, cols), dtype=np.float32)
    angles[:, 0::2] = round_bf16(rng.random((angle_rows, half)))
    angles[:, 1::2] = round_bf16(rng.random((angle_rows, half)))
    assert np.array_equal(ops.rope(x, angles), _block_major_expected(x, angles, rows, angle_rows))


def test_rope_is_a_rotation_and_interleaved_matches_complex_multiply():
    rng = np.random.default_rng(5)
    theta = rng.uniform(-np.pi, np.pi, (4, 16))
    table = np.empty((4, 32), np.float32)
    table[:, ::2], table[:, 1::2] = np.cos(theta), np.sin(theta)
    x = bf(rng, 8, 32)
    y = ops.rope(x, table)  # unrounded table: norms preserved up to the output rounding
    assert np.allclose(np.linalg.norm(y, axis=1), np.linalg.norm(x, axis=1), rtol=1e-2)
    # Interleaved pairs: (x0 + i x1) * e^{i theta}.
    yi = ops.rope(x, table, two_halves=False)
    z = (x[:, 0::2] + 1j * x[:, 1::2]).reshape(4, 2, 16) * np.exp(1j * theta)[:, None]
    want = np.empty_like(x)
    want[:, 0::2], want[:, 1::2] = z.real.reshape(8, 16), z.imag.reshape(8, 16)
    assert np.allclose(yi, want, rtol=2.0**-7, atol=1e-2)


# ------------------------------------------------------------------ elementwise
def test_add_is_bit_exact_single_rounding():
    rng = np.random.default_rng(6)
    a, b = bf(rng, 4096, scale=3), bf(rng, 4096, scale=3)
    want = round_bf16((a.astype(np.float64) + b.astype(np.float64)).astype(np.float32))
    assert np.array_equal(ops.add(a, b), want)


def test_mul_and_silu_against_float64():
    rng = np.random.default_rng(7)
    a, b = bf(rng, 4096, scale=3), bf(rng, 4096, scale=3)
    # A product of two bf16 values is exact in float32: one rounding of the exact product.
    assert np.array_equal(ops.mul(a, b), round_bf16((a.astype(np.float64) * b).astype(np.float32)))
    x64 = a.astype(np.float64)
    exact = x64 / (1 + np.exp(-x64))
    assert np.all(np.abs(ops.silu(a) - exact) <= 2.0**-7 * np.abs(exact) + 1e-30)
    assert ops.silu(np.zeros(1, np.float32))[0] == 0


def test_rms_norm_structure():
    rng = np.random.default_rng(8)
    x, w = bf(rng, 5, 256, scale=2), round_bf16(rng.uniform(0.9, 1.1, 256))
    x64 = x.astype(np.float64)
    normed = x64 / np.sqrt((x64**2).mean(-1, keepdims=True) + 1e-5)
    got = ops.rms_norm(x, epsilon=1e-5)
    assert np.all(np.abs(got - normed) <= 2.0**-7 * np.abs(normed) + 1e-6)
    # Weighted: the rounded row times the weight, rounded again (two roundings).
    assert np.array_equal(ops.rms_norm(x, w, epsilon=1e-5), round_bf16(got * w))
    # Scale invariance where eps is negligible; eps matters on a tiny row.
    assert np.allclose(ops.rms_norm(4 * x, epsilon=1e-12), ops.rms_norm(x, epsilon=1e-12), rtol=2**-6)
    tiny = np.full((1, 8), 2.0**-10, np.float32)
    assert ops.rms_norm(tiny, epsilon=1.0)[0, 0] < ops.rms_norm(tiny, epsilon=1e-12)[0, 0]


# ------------------------------------------------------------------- attention
def _brute_force_mha(Q, K, V, groups, offset, causal, window, scale):
    """Per query, per head, in float64 with explicit loops: (heads, rows, d)."""
    H, S, d = Q.shape
    out = np.zeros((H, S, d))
    for h in range(H):
        for i in range(S):
            pos = offset + i
            keep = []
            for j in range(K.shape[1]):
                if causal and j > pos:
                    continue
                if not causal and window is not None and j > pos + window:
                    continue
                if window is not None and j < pos - window:
                    continue
                keep.append(j)
            s = np.array([Q[h, i].astype(np.float64) @ K[h // groups, j] * scale for j in keep])
            p = np.exp(s - s.max())
            p /= p.sum()
            out[h, i] = sum(pj * V[h // groups, j].astype(np.float64) for pj, j in zip(p, keep))
    return out


@pytest.mark.parametrize("causal,window", [(True, None), (True, 3), (False, 2), (False, None)])
def test_mha_against_brute_force(causal, window):
    rng = np.random.default_rng(9)
    H, G, S, L, d = 4, 2, 6, 10, 8
    Q, K, V = bf(rng, H, S, d), bf(rng, G, L, d), bf(rng, G, L, d)
    scale = 1 / math.sqrt(d)
    got = ops.mha(Q, K, V, num_heads=H, num_KV_heads=G, seq_len=S, kv_len=L, d=d, causal=causal,
                  window=window, scale=scale)
    offset = L - S if (causal or window) else 0
    want = _brute_force_mha(Q, K, V, H // G, offset, causal, window, scale)
    assert np.allclose(got, want, rtol=2.0**-7, atol=1e-3)


def test_mha_layouts_bounds_and_chunking():
    rng = np.random.default_rng(10)
    H, G, L, d = 4, 2, 24, 8
    Q, K, V = bf(rng, L, H, d), bf(rng, L, G, d), bf(rng, L, G, d)
    kw = dict(num_heads=H, num_KV_heads=G, d=d, heads_interleaved=True, kv_interleaved=True)
    whole = ops.mha(Q, K, V, seq_len=L, kv_len=L, **kw)
    # Interleaved layouts are pure transposes of the head-major ones.
    hm = ops.mha(np.swapaxes(Q, 0, 1), np.swapaxes(K, 0, 1), np.swapaxes(V, 0, 1), num_heads=H,
                 num_KV_heads=G, d=d, seq_len=L, kv_len=L)
    assert np.array_equal(whole, np.swapaxes(hm, 0, 1))
    # A chunk of 8 queries over the cache equals the same rows of the whole (causal).
    for start in (0, 8, 16):
        chunk = ops.mha(Q[start : start + 8], K, V, seq_len=8, kv_len=L, valid=8,
                        kv_valid=start + 8, **kw)
        assert np.array_equal(chunk, whole[start : start + 8])
    # A bounded call: rows past the bound are exactly zero, what lies past it is never read.
    poisonK, poisonV, poisonQ = K.copy(), V.copy(), Q[8:16].copy()
    poisonK[13:], poisonV[13:], poisonQ[5:] = np.nan, np.nan, np.nan
    out = ops.mha(poisonQ, poisonK, poisonV, seq_len=8, kv_len=L, valid=5, kv_valid=13, **kw)
    assert np.array_equal(out[5:], np.zeros_like(out[5:]))
    assert np.array_equal(out[:5], whole[8:13])
    # One query (decode) is the last row of the whole.
    one = ops.mha(Q[L - 1 : L], K, V, seq_len=1, kv_len=L, kv_valid=L, **kw)
    assert np.array_equal(one[0], whole[L - 1])


# ------------------------------------------------------------------------ glue
def test_gather_and_argmax():
    table = np.arange(40, dtype=np.float32).reshape(10, 4)
    assert np.array_equal(ops.gather_rows(table, [3, 0, 3]), table[[3, 0, 3]])
    logits = np.array([1.0, 5.0, 5.0, -2.0], np.float32)
    assert ops.argmax(logits) == 1  # first of the ties


# ------------------------------------------------------- the sibling decoders' operators
# Their kernels' references live in mlir-aie (parity unpinned there); each restatement is held to a
# float64 library routine of the same function, within one rounding to bf16.
def _within_a_bf16_step(got, want64, atol=2.0**-126):
    """``atol``: what float32's own rounding leaves of a result that cancels (1 + erf(x) far in the tail)."""
    want = round_bf16(want64.astype(np.float32))
    step = np.maximum(np.abs(want) * 2.0**-7, atol)
    assert np.all(np.abs(got - want) <= step), np.abs(got - want).max()
    assert is_bf16_valued(got)


def test_activations_match_float64_library_routines():
    import torch

    rng = np.random.default_rng(30)
    x = bf(rng, 4096, scale=3.0)
    x64 = torch.from_numpy(x.astype(np.float64))
    _within_a_bf16_step(ops.gelu(x), torch.nn.functional.gelu(x64, approximate="tanh").numpy(), atol=1e-5)
    _within_a_bf16_step(ops.gelu(x, "none"), torch.nn.functional.gelu(x64).numpy(), atol=1e-5)
    _within_a_bf16_step(ops.sigmoid(x), torch.sigmoid(x64).numpy())
    _within_a_bf16_step(ops.tanh(x), np.tanh(x.astype(np.float64)))
    assert np.array_equal(ops.relu(x), np.where(x > 0, x, 0))
    # The clamp's bounds are rounded to bf16 first: 1.003 is 1.0 there.
    assert np.array_equal(ops.clamp(x, -0.75, 1.003), np.clip(x, -0.75, 1.0))
    # GELU's two forms differ where the approximation does (about 1e-3 near |x| = 2), not elsewhere.
    assert 1e-4 < np.abs(ops.gelu(x) - ops.gelu(x, "none")).max() < 2e-2


def test_axpy_is_one_fused_multiply_add():
    rng = np.random.default_rng(31)
    x, y = bf(rng, 2048, scale=4.0), bf(rng, 2048, scale=4.0)
    for a in (3.0, 1.003, -0.5):
        want = np.float32(a).astype(np.float64) * x.astype(np.float64) + y.astype(np.float64)
        _within_a_bf16_step(ops.axpy(a, x, y), want)
    # The scalar stays float32: 1.003 is not 1.0 (it would be, rounded to bf16).
    assert not np.array_equal(ops.axpy(1.003, x, y), ops.axpy(1.0, x, y))
    assert np.array_equal(ops.axpy(1.0, x, y), ops.add(x, y))


def test_layer_norm_matches_torch_in_float64():
    import torch

    rng = np.random.default_rng(32)
    x = bf(rng, 6, 1024, scale=2.0) + np.float32(1.5)   # a mean to take away
    x = round_bf16(x)
    w = round_bf16(rng.uniform(0.9, 1.1, 1024).astype(np.float32))
    x64 = torch.from_numpy(x.astype(np.float64))
    plain = torch.nn.functional.layer_norm(x64, (1024,), eps=1e-5).numpy()
    _within_a_bf16_step(ops.layer_norm(x), plain)
    # Weighted: the normalised row is rounded before the multiply (two roundings).
    assert np.array_equal(ops.layer_norm(x, w), round_bf16(ops.layer_norm(x) * w))
    # Not RMSNorm: a constant added to a row changes nothing.
    assert np.array_equal(ops.layer_norm(round_bf16(x[:1])), ops.layer_norm(x)[:1])
    shifted = ops.layer_norm(x + np.float32(8.0))
    assert np.abs(shifted - ops.layer_norm(x)).max() < 0.05 and np.abs(ops.rms_norm(x + np.float32(8.0)) - ops.rms_norm(x)).max() > 0.2


def test_softmax_matches_scipy_with_its_cap_addend_and_length():
    from scipy.special import softmax

    rng = np.random.default_rng(33)
    x = rng.normal(0, 4, (16, 512)).astype(np.float32)
    addend = rng.normal(0, 1, (16, 512)).astype(np.float32)
    _within_a_bf16_step(ops.softmax(x), softmax(x.astype(np.float64), axis=-1))
    capped = 30.0 * np.tanh((x.astype(np.float64) + addend) / 30.0)
    _within_a_bf16_step(ops.softmax(x, addend, soft_cap=30.0), softmax(capped, axis=-1))
    short = ops.softmax(x, length=100)
    _within_a_bf16_step(short[:, :100], softmax(x[:, :100].astype(np.float64), axis=-1))
    assert not short[:, 100:].any()
    assert np.allclose(ops.softmax(x).sum(axis=-1), 1.0, atol=5e-3)


# -------------------------------------------------------------------- sampling
# The draw with a temperature is this build's own definition (the reference's sample_ref is not
# in its tree), so it is pinned to what the mathematics fixes: exp, softmax, an exact cumulative walk.
def test_exp_det_is_exp_to_an_ulp():
    rng = np.random.default_rng(0)
    zs = np.concatenate([-rng.random(5000) * 40, -rng.random(500) * 690, [0.0, -0.0, -1e-300, -690.0, -0.34657359]])
    worst = max(abs(ops.exp_det(float(z)) - math.exp(z)) / math.exp(z) for z in zs)
    assert worst < 4e-16
    assert ops.exp_det(0.0) == 1.0
    assert ops.exp_det(-690.1) == 0.0 and ops.exp_det(-math.inf) == 0.0 and ops.exp_det(math.nan) == 0.0


def test_sample_order_and_greedy():
    x = np.array([1.0, 5.0, np.nan, 5.0, -np.inf, -0.0, 0.0, 7.0, 7.0], np.float32)
    # Larger first, of equals the lower index (-0 equals +0), NaN last.
    assert ops.sample_order(x).tolist() == [7, 8, 1, 3, 0, 5, 6, 4, 2]
    assert ops.sample_ref(x, 0.0, 50, 12345) == 7
    assert ops.sample_ref(x, 0.7, 1, (1 << 53) - 1) == 7          # top-1 is greedy whatever the number
    assert ops.sample_ref(x, 0.7, 50, 0) == 7                     # the number 0 draws the best
    assert ops.sample_ref(x, 1e-3, 50, (1 << 52) - 1) == 7        # u just under 1/2, two equal bests
    assert ops.sample_ref(x, 1e-3, 50, 1 << 52) == 8              # u = 1/2: the second of them
    # A best logit that is not finite draws itself; NaN and -inf candidates weigh nothing.
    assert ops.sample_ref(np.array([1.0, np.inf, 3.0], np.float32), 0.7, 3, 1 << 52) == 1
    assert ops.sample_ref(np.array([np.nan, -np.inf, 3.0], np.float32), 0.7, 3, (1 << 53) - 1) == 2


def test_sample_weights_are_the_top_k_softmax():
    from scipy.special import softmax

    rng = np.random.default_rng(5)
    x = round_bf16(rng.normal(0, 3, 2000))
    for t, k in [(0.7, 50), (1.0, 7), (0.05, 64), (5.0, 33)]:
        cand, w = ops.sample_weights(x, t, k)
        assert cand.tolist() == sorted(range(x.size), key=lambda i: (-x[i], i))[:k]
        want = softmax(x[cand].astype(np.float64) / float(np.float32(t)))
        assert np.allclose(w / w.sum(), want, rtol=1e-13, atol=0)
    # k_max caps top_k; a top_k past the row keeps the row.
    assert ops.sample_weights(x, 0.7, 500, k_max=64)[0].size == 64
    assert ops.sample_weights(x[:10], 0.7, 50)[0].size == 10


def test_sample_ref_walks_the_cumulative_weights():
    from fractions import Fraction

    rng = np.random.default_rng(6)
    x = round_bf16(rng.normal(0, 2, 512))
    x[[3, 77, 78]] = x.max()   # ties at the top, in index order
    for t, k in [(0.7, 50), (1.5, 64), (0.3, 5)]:
        cand, w = ops.sample_weights(x, t, k)
        cum = np.cumsum([Fraction(float(v)) for v in w])
        seen = set()
        for n53 in rng.integers(0, 1 << 53, 400):
            u = Fraction(int(n53), 1 << 53)
            want = next(i for i, c in enumerate(cum) if c > u * cum[-1])
            got = ops.sample_ref(x, t, k, int(n53))
            assert got == cand[want]
            seen.add(want)
        assert len(seen) > 1
        # Either side of the first boundary: the number just under w0/total draws the best, the
        # next but one draws its neighbour.
        edge = int(Fraction(float(w[0])) / cum[-1] * (1 << 53))
        assert ops.sample_ref(x, t, k, edge - 1) == cand[0]
        assert ops.sample_ref(x, t, k, edge + 1) == cand[1]


def test_draw_row_words_round_trip():
    from iron_amd.operators.sample import draw_row

    row = draw_row(0.7, 50, (1 << 53) - 12345)
    assert row.dtype == np.int32 and row.shape == (4,)
    t, k, n = ops.draw_words(row)
    assert t == np.float32(0.7) and k == 50 and n == (1 << 53) - 12345
    assert ops.draw_words(np.zeros(4, np.int32)) == (0.0, 1, 0)
    with pytest.raises(ValueError, match="53-bit"):
        draw_row(0.7, 50, 1 << 53)


def test_sampler_draws_what_its_rows_draw():
    import oracle
    from iron_amd.lm.generation import Sampler

    oracle.install()
    rng = np.random.default_rng(8)
    x = round_bf16(rng.normal(0, 3, 4096))
    host, device = Sampler(0.7, 50, seed=3), Sampler(0.7, 50, seed=3)
    rows = device.rows(20, 64)
    for r in rows:
        assert host(x) == ops.sample_ref(x, *ops.draw_words(r), 64)
    probs = Sampler(0.7, 50).probabilities(x)
    assert abs(probs.sum() - 1) < 1e-12 and np.count_nonzero(probs) == 50
    assert Sampler(0.0, 50).probabilities(x).argmax() == x.argmax()
    with pytest.raises(ValueError, match="not one the device draws"):
        Sampler(0.7, None).rows(1, 64)
    with pytest.raises(ValueError, match="below zero"):
        Sampler(-1.0)


# ----------------------------------------------------------------- RoPE tables
def test_rope_angles_closed_forms():
    t = ops.rope_angles(64, 128, 500000.0)
    assert t.shape == (128, 64) and t.dtype == np.float32
    # Row 0 is (cos 0, sin 0) pairs; pair j of row p is the angle p * theta^(-2j/64).
    assert np.array_equal(t[0, 0::2], np.ones(32, np.float32))
    assert np.array_equal(t[0, 1::2], np.zeros(32, np.float32))
    # float32 frequency times float32 position, cos/sin in float64, rounded once
    # (the statement of iron/tests/infrastructure/test_rope_angles.py:20-37).
    p, j = 37, 5
    inv = np.float32(1.0 / 500000.0 ** np.float64(np.float32(2 * j) / np.float32(64)))
    ang = np.float64(np.float32(p) * inv)
    assert t[p, 2 * j] == np.float32(np.cos(ang)) and t[p, 2 * j + 1] == np.float32(np.sin(ang))
    # And within float32 rounding of the formula in float64 throughout.
    exact_freqs = np.outer(np.arange(128), 1.0 / 500000.0 ** (np.arange(0, 64, 2) / 64))
    exact = np.empty((128, 64))
    exact[:, ::2], exact[:, 1::2] = np.cos(exact_freqs), np.sin(exact_freqs)
    assert np.abs(t - exact).max() < 5e-4
    assert np.allclose(t[:, 0::2] ** 2 + t[:, 1::2] ** 2, 1.0, atol=1e-6)


def test_llama3_scaling_bands():
    scale = ops.llama3_scaling(8.0, 1.0, 4.0, 64)
    exps = np.arange(0, 64, 2, dtype=np.float32) / np.float32(64)
    inv = 1.0 / np.power(500000.0, exps.astype(np.float64))
    out = scale(inv)
    wavelen = 2 * np.pi / inv
    high, low = wavelen < 64 / 4.0, wavelen > 64 / 1.0
    assert np.array_equal(out[high], inv[high])
    assert np.allclose(out[low], inv[low] / 8.0)
    mid = ~high & ~low
    assert mid.any() and np.all(out[mid] < inv[mid]) and np.all(out[mid] > inv[mid] / 8.0)


def test_filled_random_draw_order_and_scales():
    named = {"a.weight": (8, 16), "b.weight": (16,), "c.bias": (16,)}
    w = ops.filled(named, seed=0)
    rng = np.random.default_rng(0)
    a = rng.standard_normal((8, 16), dtype=np.float32)
    b = rng.standard_normal((16,), dtype=np.float32)
    c = rng.standard_normal((16,), dtype=np.float32)
    assert np.array_equal(w["a.weight"], round_bf16((a / 4.0).astype(np.float32)))
    assert np.array_equal(w["b.weight"], round_bf16(b / 10 + 1))
    assert np.array_equal(w["c.bias"], round_bf16(c / 10))

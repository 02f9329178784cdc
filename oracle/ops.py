"""CPU restatement of the reference operators' ``reference()`` methods.

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, by ``__graft_entry__.smoke``
and by ``bench.py``'s cpu_baseline leg as the checker; the product package
never imports it.

Conventions: a bf16 operand is a float32 numpy array whose values are exactly
representable in bf16 (``iron_amd.bf16``); every function computes in float32
as the reference does and rounds once to bf16 where the reference casts
``astype(bfloat16)``.

Pinned by (see tests/test_oracle.py):
  gemm        f64 matmul + one rounding; tolerance formula      gemm.py:696-735
  gemv        f64 matvec + one rounding                          gemv.py:408-421
  rope        closed form row by row, array_equal                test_rope_reference_convention.py:27-64
  mha         brute force per query on tiny inputs, chunk-vs-whole,
              padding rows zero                                  mha.py:1073-1116, test_mha_bounded_rows.py
  add         bit-exact bf16(f32(a)+f32(b))                      test_elementwise.py:125-132
  copy/gather exact                                              copy.py:839-902
  argmax      np.argmax of f32 logits (first of ties)            sample.py:72-79
  rope_angles closed forms                                       test_rope_angles.py:20-107
  sample_ref  (temperature > 0) against what the mathematics fixes: exp_det
              against math.exp, the draw's distribution against softmax
              of the top-k logits / T, the cumulative walk against exact
              rationals, top_k = 1 / n53 = 0 = greedy
Parity unpinned (arithmetic lives in mlir-aie 1.4.6.dev15, absent here; textbook
formula used, bounded by the stated bf16 tolerance and the model-level goldens):
  rms_norm inner summation order / rsqrt, silu (LUT kernel), mul; gelu, sigmoid, tanh (table
  kernels), axpy, layer_norm, softmax -- each checked against a float64 library routine instead;
  sample_ref with temperature > 0 (aie.iron.kernels.sample.sample_ref): which token
  a given 53-bit number draws is this build's own definition, stated at sample_ref.
"""

from __future__ import annotations

import math

import numpy as np

from iron_amd.bf16 import round_bf16


def _f32(x):
    return np.asarray(x, dtype=np.float32)


# ---------------------------------------------------------------- GEMM / GEMV


def gemm(A, B, *, b_col_maj=False, c_col_maj=False, valid_k=None):
    """``A @ B`` in float32 over the first ``valid_k`` of K, rounded once (gemm.py:696-702)."""
    a = _f32(A)
    K = a.shape[1]
    valid_k = K if valid_k is None else int(valid_k)
    a = a[:, :valid_k]
    b = (_f32(B).T if b_col_maj else _f32(B))[:valid_k]
    C = np.matmul(b.T, a.T) if c_col_maj else np.matmul(a, b)
    return round_bf16(C)


def gemm_bound(A, B, *, b_col_maj=False, c_col_maj=False, units=2.0):
    """The admitted |error| of GEMM at HIGHEST: ``units`` · 2^-8 · |A|@|B| (gemm.py:704-735)."""
    a = _f32(A)
    b = _f32(B).T if b_col_maj else _f32(B)
    err = units * (np.abs(a) @ np.abs(b)) * 2.0**-8
    return err.T if c_col_maj else err


def gemv(A, B, *, repeat=1):
    """``C = A @ B``, one product per batch, float32, rounded once (gemv.py:408-417)."""
    A, B = _f32(A), _f32(B)
    if repeat > 1:
        A = np.repeat(A.reshape(-1, *A.shape[-2:]), repeat, axis=0)
    if A.ndim == 3:
        b = B.reshape(A.shape[0], A.shape[2], 1)
        return round_bf16(np.matmul(A, b).reshape(A.shape[0], A.shape[1]))
    return round_bf16(A @ B.reshape(A.shape[-1]))


# ------------------------------------------------------------ rowwise / eltwise


def rms_norm(x, weight=None, *, epsilon=1e-5):
    """Each row over its RMS, rounded to bf16; then times ``weight``, rounded again.

    Structure from elementwise.py:676-682 (the norm's row is rounded before the
    multiply); the row formula ``x * 1/sqrt(mean(x^2) + eps)`` is the textbook one
    (flm/layer/reference.py:108-119 hints the same) -- parity unpinned.
    """
    x = _f32(x)
    ms = np.mean(x * x, axis=-1, keepdims=True, dtype=np.float32)
    inv = (np.float32(1.0) / np.sqrt(ms + np.float32(epsilon))).astype(np.float32)
    normed = round_bf16(x * inv)
    if weight is None:
        return normed
    return round_bf16(normed * _f32(weight).reshape(-1))


def silu(x):
    """``x * sigmoid(x)`` in float32, rounded once (silu.py:12; LUT kernel -- parity unpinned)."""
    x = _f32(x)
    return round_bf16(x / (np.float32(1.0) + np.exp(-x)))


def gelu(x, approximate="tanh"):
    """GELU in float32, rounded once: ``0.5 x (1 + tanh(sqrt(2/pi)(x + 0.044715 x^3)))``, or exact
    ``x Phi(x)`` (gelu.py:13-40, torch's ``approximate``; the reference's kernels are a table and an
    erf of mlir-aie -- parity unpinned)."""
    x = _f32(x)
    if approximate == "none":
        from scipy.special import erf

        return round_bf16(np.float32(0.5) * x * (np.float32(1.0) + erf(x * np.float32(0.7071067811865476)).astype(np.float32)))
    inner = np.float32(0.7978845608028654) * (x + np.float32(0.044715) * x * x * x)
    return round_bf16(np.float32(0.5) * x * (np.float32(1.0) + np.tanh(inner)))


def relu(x):
    """``max(x, 0)`` (relu.py:11; pinned bit-exact with an add by test_elementwise.py:125-132)."""
    return np.maximum(_f32(x), np.float32(0.0))


def sigmoid(x):
    """``1 / (1 + exp(-x))`` in float32, rounded once (sigmoid.py:9; table kernel -- parity unpinned)."""
    return round_bf16(np.float32(1.0) / (np.float32(1.0) + np.exp(-_f32(x))))


def tanh(x):
    """``tanh(x)`` in float32, rounded once (tanh.py:9; table kernel -- parity unpinned)."""
    return round_bf16(np.tanh(_f32(x)))


def clamp(x, low, high):
    """``x`` clamped to ``[low, high]``, the bounds rounded to bf16 (clamp.py:14-63): exact."""
    lo, hi = round_bf16(np.array([low, high], np.float32))
    return np.minimum(np.maximum(_f32(x), lo), hi)


def axpy(a, x, y):
    """``a x + y``: the product exact in float64, the sum rounded to float32 (a fused multiply-add),
    then to bf16 (axpy.py:13-31 over datamovement.axpy -- parity unpinned)."""
    fused = (np.float64(np.float32(a)) * _f32(x).astype(np.float64) + _f32(y).astype(np.float64)).astype(np.float32)
    return round_bf16(fused)


def layer_norm(x, weight=None, *, epsilon=1e-5):
    """Each row less its mean over its standard deviation (beta 0), rounded to bf16; then times
    ``weight``, rounded again (layer_norm.py:10-20; structure from elementwise.py:676-682; the row
    formula is the textbook one, torch's -- parity unpinned)."""
    x = _f32(x)
    mean = np.mean(x, axis=-1, keepdims=True, dtype=np.float32)
    centred = x - mean
    var = np.mean(centred * centred, axis=-1, keepdims=True, dtype=np.float32)
    normed = round_bf16(centred * (np.float32(1.0) / np.sqrt(var + np.float32(epsilon))).astype(np.float32))
    if weight is None:
        return normed
    return round_bf16(normed * _f32(weight).reshape(-1))


def softmax(x, addend=None, *, soft_cap=None, length=None):
    """Softmax of each row over its first ``length`` columns, the rest zero (softmax.py:523-545 over
    activation.softmax_ref -- parity unpinned): ``z = x + addend``, capped as ``cap tanh(z / cap)``,
    ``exp(z - max) / sum`` in float32, one rounding."""
    x = np.asarray(x, dtype=np.float32)
    n = x.shape[-1] if length is None else int(length)
    z = x[..., :n]
    if addend is not None:
        z = z + np.asarray(addend, dtype=np.float32)[..., :n]
    if soft_cap is not None:
        z = np.float32(soft_cap) * np.tanh(z / np.float32(soft_cap))
    e = np.exp(z - z.max(axis=-1, keepdims=True))
    out = np.zeros(x.shape, np.float32)
    out[..., :n] = round_bf16(e / e.sum(axis=-1, keepdims=True, dtype=np.float32))
    return out


def mul(a, b):
    """``bf16(f32(a) * f32(b))`` (elementwise_mul.py:11)."""
    return round_bf16(_f32(a) * _f32(b))


def add(a, b):
    """``bf16(f32(a) + f32(b))`` (elementwise_add.py:11; test_elementwise.py:125-132)."""
    return round_bf16(_f32(a) + _f32(b))


def rope(x, angles, *, two_halves=True):
    """Rotate each row of ``x`` by its angle row; row r uses angle row ``r // (rows/angle_rows)``.

    ``angles`` is the packed bf16 table, cos and sin interleaved (rope.py:167-184).
    two_halves=False (interleaved pairs) is the textbook pair rotation -- parity unpinned.
    """
    x, angles = _f32(x), _f32(angles)
    rows, cols, lut_rows = x.shape[0], x.shape[-1], angles.shape[0]
    if rows % lut_rows:
        raise ValueError(f"RoPE: angles ({lut_rows} rows) must divide x's {rows} rows")
    xr = x.reshape(lut_rows, -1, cols)
    cos = angles[:, None, 0::2]
    sin = angles[:, None, 1::2]
    y = np.empty_like(xr)
    if two_halves:
        h = cols // 2
        x1, x2 = xr[..., :h], xr[..., h:]
        y[..., :h] = x1 * cos - x2 * sin
        y[..., h:] = x2 * cos + x1 * sin
    else:
        x1, x2 = xr[..., 0::2], xr[..., 1::2]
        y[..., 0::2] = x1 * cos - x2 * sin
        y[..., 1::2] = x2 * cos + x1 * sin
    return round_bf16(y.reshape(x.shape))


# ------------------------------------------------------------------- attention


def mha(
    Q,
    K,
    V,
    *,
    num_heads,
    num_KV_heads=None,
    seq_len=None,
    kv_len=None,
    d=64,
    causal=True,
    window=None,
    scale=None,
    heads_interleaved=False,
    kv_interleaved=False,
    valid=None,
    kv_valid=None,
):
    """Attention per head, the queries the keys' last rows (mha.py:1073-1116).

    ``valid`` / ``kv_valid`` are a bounded call's rows and keys; query rows past
    the bound come out zero and keys past it are dropped.
    """
    Q, K, V = _f32(Q), _f32(K), _f32(V)
    num_KV_heads = num_heads if num_KV_heads is None else num_KV_heads
    if heads_interleaved:
        Q = np.swapaxes(Q, 0, 1)
    if kv_interleaved:
        K, V = np.swapaxes(K, 0, 1), np.swapaxes(V, 0, 1)
    seq_pad = Q.shape[1]
    seq_len = seq_pad if seq_len is None else seq_len
    kv_len = K.shape[1] if kv_len is None else kv_len
    scale = float(1 / np.sqrt(d)) if scale is None else scale
    q_tokens = seq_len if valid is None else int(valid)
    kv_tokens = (kv_len - seq_pad + q_tokens) if kv_valid is None else int(kv_valid)
    groups = num_heads // num_KV_heads
    offset = kv_tokens - q_tokens
    if (causal or window) and offset < 0:
        raise ValueError(f"MHA: the {q_tokens} queries are more than the {kv_tokens} keys")
    start = offset if causal or window else 0
    s_q = start + q_tokens
    K, V = K[:, :kv_tokens], V[:, :kv_tokens]
    rows = max(s_q - start, 0)
    q = Q[:, :rows]
    key = np.arange(K.shape[1])
    scale = np.float32(scale)
    out = np.zeros(Q.shape, dtype=np.float32)
    step = max(1, 2**24 // max(K.shape[1], 1))
    for first in range(0, rows, step):
        block = slice(first, min(first + step, rows))
        position = offset + np.arange(block.start, block.stop)[:, None]
        masked = np.zeros((len(position), K.shape[1]), dtype=bool)
        if causal or window:
            masked |= key > position + (0 if causal else (window or 0))
        if window:
            masked |= key < position - window
        mask = np.where(masked, -np.inf, 0).astype(np.float32)
        for h in range(q.shape[0]):
            scores = q[h, block] @ K[h // groups].T * scale + mask
            e = np.exp(scores - scores.max(axis=-1, keepdims=True))
            out[h, block] = round_bf16((e / e.sum(axis=-1, keepdims=True)) @ V[h // groups])
    if heads_interleaved:
        return np.ascontiguousarray(np.swapaxes(out, 0, 1))
    return out


# --------------------------------------------------------------------- glue


def gather_rows(table, ids):
    """Rows of ``table`` named by ``ids`` (copy.py:839-902: exact)."""
    return np.asarray(table)[np.asarray(ids, dtype=np.int64)]


def argmax(logits) -> int:
    """Greedy draw: the first largest float32 logit (sample.py:72-79, test_lm_host.py:554-557)."""
    return int(np.argmax(_f32(logits).reshape(-1)))


# ------------------------------------------------------------------ sampling

LOG2E = 1.4426950408889634
LN2_HI = 6.93147180369123816490e-01   # ln 2 with its low 32 bits zero: n * LN2_HI is exact for |n| < 2**20
LN2_LO = 1.90821492927058770002e-10
EXP_FLOOR = -690.0                    # below it a weight is 0.0
EXP_COEFFS = [1.0 / math.factorial(i) for i in range(14)]


def exp_det(z: float) -> float:
    """``exp(z)`` for ``z <= 0`` from IEEE double +, -, * alone (no fused multiply-add, no library
    exp), so that any machine computes the same bits: n = rint(z * log2 e), r = z - n ln 2 in two
    steps, a degree-13 Taylor polynomial by Horner, an exact scaling by 2**n."""
    if not z >= EXP_FLOOR:   # also NaN
        return 0.0
    n = float(round(z * LOG2E))   # round(): half to even, as rint
    r = (z - n * LN2_HI) - n * LN2_LO
    p = EXP_COEFFS[13]
    for c in EXP_COEFFS[12::-1]:
        p = p * r + c
    return math.ldexp(p, int(n))


def sample_order(logits) -> np.ndarray:
    """The indices of ``logits`` from the best: larger first, of equals the lower index, NaN last."""
    x = _f32(logits).reshape(-1)
    key = np.where(np.isnan(x), -np.inf, x).astype(np.float64)
    nan = np.isnan(x)
    # lexsort: the last key is the primary one.
    return np.lexsort((np.arange(x.size), -key, nan))


def sample_weights(logits, temperature, top_k, k_max=None):
    """``(candidates, weights)``: the ``top_k`` best tokens (at most ``k_max``) in ``sample_order``
    and each one's weight ``exp_det((logit - best) / temperature)`` in float64, 0.0 for a NaN logit."""
    x = _f32(logits).reshape(-1)
    k = min(max(int(top_k), 1), x.size if k_max is None else min(int(k_max), x.size))
    cand = sample_order(x)[:k]
    top, t = float(x[cand[0]]), float(np.float32(temperature))
    weights = np.array([0.0 if math.isnan(float(x[i])) else exp_det((float(x[i]) - top) / t) for i in cand])
    return cand, weights


def sample_ref(logits, temperature, top_k, n53, k_max=None) -> int:
    """The token a draw row draws from a row of bf16 logits (iron/operators/sample.py:72-79's
    ``sample.sample_ref``, whose arithmetic is not in the reference's tree: this is the
    definition this build's device kernel follows, bit for bit).

    A temperature that is not positive is greedy: the first largest logit.  Otherwise the candidates are the
    ``top_k`` (1..``k_max``) best logits, ties to the lower index; candidate i weighs
    ``exp_det((l_i - l_0) / T)`` in float64 (T the float32 temperature); with ``total`` the
    weights summed in candidate order and ``threshold = (n53 * 2**-53) * total``, the draw
    is the first candidate whose running sum exceeds the threshold (the last of non-zero
    weight if rounding leaves none).  A best logit that is not finite draws itself.
    """
    x = _f32(logits).reshape(-1)
    if not float(np.float32(temperature)) > 0.0:
        return int(sample_order(x)[0])
    cand, weights = sample_weights(x, temperature, top_k, k_max)
    if not math.isfinite(float(x[cand[0]])):
        return int(cand[0])
    total = 0.0
    for w in weights:
        total += float(w)
    threshold = (float(int(n53)) * 2.0 ** -53) * total
    running, last = 0.0, 0
    for i, w in enumerate(weights):
        running += float(w)
        if running > threshold:
            return int(cand[i])
        if w > 0.0:
            last = i
    return int(cand[last])


def draw_words(draw_row):
    """``(temperature, top_k, n53)`` of a four-word draw row (iron/operators/sample.py:72-79)."""
    words = np.asarray(draw_row, dtype=np.int32).reshape(-1)
    row = words.view(np.uint32)
    temperature = row[0:1].view(np.float32)[0]
    return temperature, max(int(words[1]), 1), (int(row[2]) | int(row[3]) << 32) & ((1 << 53) - 1)


# --------------------------------------------------------------- RoPE tables


def rope_angles(head_dim, context_length, rope_theta=500000.0, scaling=None):
    """The RoPE table ``(context_length, head_dim)`` float32, cos/sin interleaved (lm/config.py:23-42)."""
    exponents = np.arange(0, head_dim, 2, dtype=np.float32) / np.float32(head_dim)
    inv_freq = 1.0 / np.power(rope_theta, exponents.astype(np.float64))
    if scaling is not None:
        inv_freq = scaling(inv_freq)
    inv_freq = inv_freq.astype(np.float32)
    freqs = np.outer(np.arange(context_length, dtype=np.float32), inv_freq)
    angles = np.empty((context_length, head_dim), dtype=np.float32)
    angles[:, ::2] = np.cos(freqs.astype(np.float64))
    angles[:, 1::2] = np.sin(freqs.astype(np.float64))
    return angles


def llama3_scaling(factor, low_freq_factor, high_freq_factor, original_max_position_embeddings):
    """Llama 3's RoPE frequency scaling (applications/llama/model.py:22-69)."""

    def scale(inv_freq):
        original = original_max_position_embeddings
        wavelen = 2 * np.pi / inv_freq
        smooth = (original / wavelen - low_freq_factor) / (high_freq_factor - low_freq_factor)
        between = (1 - smooth) * inv_freq / factor + smooth * inv_freq
        return np.where(
            wavelen < original / high_freq_factor,
            inv_freq,
            np.where(wavelen > original / low_freq_factor, inv_freq / factor, between),
        )

    return scale


# ------------------------------------------------------------- random weights


def filled(named, seed=0):
    """Weights from their shapes alone: ``filled("random", ...)`` (common/graph/fill.py:13-33), bf16."""
    rng = np.random.default_rng(seed)
    out = {}
    for n, shape in named.items():
        x = rng.standard_normal(shape, dtype=np.float32)
        if len(shape) >= 2:
            # numpy >= 2: float32 array / np.float64 scalar divides in float64.
            out[n] = round_bf16((x / np.sqrt(float(np.prod(shape[1:])))).astype(np.float32))
        else:
            out[n] = round_bf16(x / 10 + (not n.endswith("bias")))
    return out

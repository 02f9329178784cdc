"""The operators' ``reference()`` methods, restated on ``oracle.ops`` -- TEST INFRASTRUCTURE.

``install()`` registers one function per operator class into
``iron_amd.common.declare.REFERENCES``; each takes the constructed operator and its
inputs as numpy arrays, as the reference's methods do (file:line cited per function).
"""

from __future__ import annotations

import numpy as np

from . import ops


def gemm(op, A, B):
    """iron/operators/gemm.py:696-702."""
    return ops.gemm(A, B, b_col_maj=op.b_col_maj, c_col_maj=op.c_col_maj, valid_k=op.valid_k)


def gemv(op, A, B):
    """iron/operators/gemv.py:408-417."""
    return ops.gemv(A, B, repeat=op.repeat)


def rms_norm(op, x, weight=None):
    """iron/common/elementwise.py:676-682 over norm.rms_norm_eps."""
    return ops.rms_norm(np.asarray(x).reshape(op.rows, op.tile_size), weight, epsilon=op.epsilon)


def silu(op, x):
    return ops.silu(x)


def mul(op, a, b):
    return ops.mul(a, np.asarray(b).reshape(np.shape(a)))


def add(op, a, b):
    return ops.add(a, np.asarray(b).reshape(np.shape(a)))


def gelu(op, x):
    """iron/operators/gelu.py:13-40."""
    return ops.gelu(x, op.approximate)


def relu(op, x):
    return ops.relu(x)


def sigmoid(op, x):
    return ops.sigmoid(x)


def tanh(op, x):
    return ops.tanh(x)


def clamp(op, x):
    """iron/operators/clamp.py:14-63."""
    return ops.clamp(x, op.low, op.high)


def axpy(op, a, b):
    """iron/operators/axpy.py:13-31: ``scalar_factor * a + b``."""
    return ops.axpy(op.scalar_factor, a, np.asarray(b).reshape(np.shape(a)))


def layer_norm(op, x, weight=None):
    """iron/common/elementwise.py:676-682 over norm.layer_norm_eps."""
    return ops.layer_norm(np.asarray(x).reshape(op.rows, op.tile_size), weight, epsilon=op.epsilon)


def softmax(op, x, addend=None):
    """iron/operators/softmax.py:523-545; a bounded call's ``length`` read off the operator."""
    length = vars(op).get("_extents", {}).get("length")
    return ops.softmax(np.asarray(x).reshape(op.rows, op.cols),
                       None if addend is None else np.asarray(addend).reshape(op.rows, op.cols),
                       soft_cap=op.soft_cap, length=length)


def rowwise_add(op, x, row):
    """iron/common/elementwise.py:797-867 over eltwise.add_sized: every row plus the one row."""
    x = np.asarray(x).reshape(op.rows, op.tile_size)
    return ops.add(x, np.broadcast_to(np.asarray(row).reshape(1, -1), x.shape))


def rowwise_mul(op, x, row):
    """iron/common/elementwise.py:797-867 over eltwise.mul_sized."""
    x = np.asarray(x).reshape(op.rows, op.tile_size)
    return ops.mul(x, np.broadcast_to(np.asarray(row).reshape(1, -1), x.shape))


def rope(op, x, angles):
    """iron/operators/rope.py:167-184; with a row wider than the table, the first columns turn and the
    rest pass through (the reference's Attention.rotate, iron/lm/blocks.py:612-620)."""
    x = np.asarray(x)
    if op.row == op.cols:
        return ops.rope(x, angles, two_halves=op.two_halves)
    y = np.array(x, dtype=np.float32).reshape(op.rows, op.row)
    y[:, : op.cols] = ops.rope(y[:, : op.cols], angles, two_halves=op.two_halves)
    return y


def mha(op, Q, K, V):
    """iron/operators/mha.py:1073-1116; a bounded call's extents read off the operator."""
    ext = vars(op).get("_extents", {})
    return ops.mha(Q, K, V, num_heads=op.num_heads, num_KV_heads=op.num_KV_heads, seq_len=op.seq_len,
                   kv_len=op.kv_len, d=op.d, causal=op.causal, window=op.window, scale=op.scale,
                   heads_interleaved=op.heads_interleaved, kv_interleaved=op.kv_interleaved,
                   valid=ext.get("valid"), kv_valid=ext.get("kv_valid"))


def copy(op, src):
    """iron/operators/copy.py:839-902: exact."""
    return np.array(src).reshape(op.shape)


def gather(op, table, control, *, valid_rows=None):
    """iron/operators/copy.py:72-378: the rows of ``table`` the first ``rows`` control words name;
    rows past ``valid_rows`` are not written (zeros here)."""
    ids = np.asarray(control).reshape(-1)[: op.rows].astype(np.int64)
    n = op.rows if valid_rows is None else int(valid_rows)
    y = np.zeros((op.rows, op.row), np.asarray(table).dtype)
    y[:n] = np.asarray(table).reshape(op.table_rows, op.row)[ids[:n]]
    return y


def gather_words(op, ids, *, valid_rows=None, base_lo=0, base_hi=0):
    """iron/operators/copy.py:380-470 as this build defines it: the ids themselves, first in ``control``."""
    control = np.zeros(op.words, np.int32)
    n = op.rows if valid_rows is None else int(valid_rows)
    control[:n] = np.asarray(ids).reshape(-1)[:n]
    return control


def sample(op, logits, draws, tokens, *, row=0, at=0):
    """iron/operators/sample.py:72-79,324-333: the draw at ``draws`` word ``row``, recorded at ``at``."""
    words = np.asarray(draws).reshape(-1)[row : row + 4]
    temperature, top_k, n53 = ops.draw_words(words)
    token = ops.sample_ref(np.asarray(logits).reshape(-1)[: op.drawable], temperature, top_k, n53, op.k_max)
    tokens = np.array(tokens, dtype=np.int32).reshape(-1)
    tokens[at] = token
    return tokens, np.array([token], dtype=np.int32)


def install() -> None:
    from iron_amd.common.declare import REFERENCES

    REFERENCES.update(
        GEMM=gemm, GEMV=gemv, RMSNorm=rms_norm, SiLU=silu, ElementwiseMul=mul, ElementwiseAdd=add,
        RoPE=rope, MHA=mha, Copy=copy, Gather=gather, GatherWords=gather_words, Sample=sample, RowwiseAdd=rowwise_add, RowwiseMul=rowwise_mul,
        GELU=gelu, ReLU=relu, Sigmoid=sigmoid, Tanh=tanh, Clamp=clamp, AXPY=axpy, LayerNorm=layer_norm,
        Softmax=softmax,
        # The host's draw, for iron_amd.lm.generation.Sampler's checks.
        sample_ref=ops.sample_ref, sample_weights=ops.sample_weights,
    )

"""Thin, typed Python calls onto the C ABI: torch CUDA tensors in, launches out.

Each function checks what the C side cannot see (dtype, device, contiguity,
element counts), passes raw device pointers and the current HIP stream, and
raises ``IronHipError`` on refusal.  Nothing here computes.
"""

from __future__ import annotations

import math

import torch

from ._lib import check, current_stream, lib, ptr

BF16 = torch.bfloat16


def _dev(t, name, dtype=BF16):
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name}: expected a torch tensor, got {type(t).__name__}")
    if not t.is_cuda:
        raise TypeError(f"{name}: expected a tensor on the GPU, got {t.device}")
    if dtype is not None and t.dtype != dtype:
        raise TypeError(f"{name}: expected {dtype}, got {t.dtype}")
    if not t.is_contiguous():
        raise ValueError(f"{name}: expected a contiguous tensor")
    return t


def _word(t, name):
    """An optional per-call word: a 1-element int32 device tensor, or None."""
    if t is None:
        return None
    _dev(t, name, torch.int32)
    if t.numel() < 1:
        raise ValueError(f"{name}: expected at least one int32 word")
    return t


def _numel(t, n, name):
    if t.numel() != n:
        raise ValueError(f"{name}: expected {n} elements, got {t.numel()} {tuple(t.shape)}")


def gemm(A, B, C, *, M, N, K, b_col_maj=False, c_col_maj=False, valid=None, valid_k=None):
    _numel(_dev(A, "A"), M * K, "A")
    _numel(_dev(B, "B"), K * N, "B")
    _numel(_dev(C, "C"), M * N, "C")
    check(
        lib().iron_gemm_bf16(
            ptr(A), ptr(B), ptr(C), M, N, K, int(b_col_maj), int(c_col_maj),
            ptr(_word(valid, "valid")), ptr(_word(valid_k, "valid_k")), current_stream(),
        ),
        "iron_gemm_bf16",
    )


def gemv(W, x, y, *, M, K, batches=1, repeat=1, valid=None, rows_per_wave=0, k_split=0):
    _numel(_dev(W, "A"), (batches // repeat) * M * K, "A")
    _numel(_dev(x, "B"), batches * K, "B")
    _numel(_dev(y, "C"), batches * M, "C")
    check(
        lib().iron_gemv_bf16_tuned(
            ptr(W), ptr(x), ptr(y), M, K, batches, repeat, ptr(_word(valid, "valid")),
            rows_per_wave, k_split, current_stream(),
        ),
        "iron_gemv_bf16",
    )


def gemm_residual(A, B, R, C, *, M, N, K, residual_scale=1.0, valid=None):
    """``C = residual_scale * (A @ B.T) + R`` over many rows, B stored ``(N, K)``."""
    _numel(_dev(A, "A"), M * K, "A")
    _numel(_dev(B, "B"), N * K, "B")
    _numel(_dev(R, "R"), M * N, "R")
    _numel(_dev(C, "C"), M * N, "C")
    check(lib().iron_gemm_residual_bf16(ptr(A), ptr(B), ptr(R), ptr(C), M, N, K, float(residual_scale),
                                        ptr(_word(valid, "valid")), current_stream()), "iron_gemm_residual_bf16")


def gemm_residual_norm_workspace_bytes(M, N, K) -> int:
    """Bytes of workspace ``gemm_residual_norm`` needs; 0 for a shape it refuses."""
    return int(lib().iron_gemm_residual_norm_workspace_bytes(M, N, K))


def gemm_residual_norm(A, B, R, gain, C, Y, workspace, *, M, N, K, eps, residual_scale=1.0, valid=None):
    """``C = residual_scale * (A @ B.T) + R`` and ``Y = rmsnorm(C) * gain`` over few rows and a long K:
    K dealt over several blocks a tile while the bound leaves the chip idle, float32 sums in
    ``workspace`` (any contents), the rows finished and normed by a second launch."""
    _numel(_dev(A, "A"), M * K, "A")
    _numel(_dev(B, "B"), N * K, "B")
    _numel(_dev(R, "R"), M * N, "R")
    _numel(_dev(gain, "gain"), N, "gain")
    _numel(_dev(C, "C"), M * N, "C")
    _numel(_dev(Y, "Y"), M * N, "Y")
    need = gemm_residual_norm_workspace_bytes(M, N, K)
    if need and _dev(workspace, "workspace", None).numel() * workspace.element_size() < need:
        raise ValueError(f"gemm_residual_norm: workspace holds {workspace.numel() * workspace.element_size()} bytes, "
                         f"{need} needed")
    check(lib().iron_gemm_residual_norm_bf16(ptr(A), ptr(B), ptr(R), ptr(gain), ptr(C), ptr(Y), M, N, K,
                                             float(residual_scale), float(eps), ptr(_word(valid, "valid")),
                                             ptr(workspace), current_stream()), "iron_gemm_residual_norm_bf16")


def gemm_gated(A, B, G, C, *, M, N, K, activation="silu", valid=None):
    """``C = act(G) * (A @ B.T)`` over many rows, B stored ``(N, K)``; ``activation`` "silu" or
    "gelu_tanh"."""
    kinds = {"silu": 1, "gelu_tanh": 2}
    if activation not in kinds:
        raise ValueError(f"gemm_gated: activation {activation!r} is neither 'silu' nor 'gelu_tanh'")
    _numel(_dev(A, "A"), M * K, "A")
    _numel(_dev(B, "B"), N * K, "B")
    _numel(_dev(G, "G"), M * N, "G")
    _numel(_dev(C, "C"), M * N, "C")
    check(lib().iron_gemm_gated_bf16(ptr(A), ptr(B), ptr(G), ptr(C), M, N, K, kinds[activation],
                                     ptr(_word(valid, "valid")), current_stream()), "iron_gemm_gated_bf16")


def gemm_gated_pair(A, Bg, Bu, G, C, *, M, N, K, activation="silu", valid=None):
    """``G = A @ Bg.T``, ``C = act(G) * (A @ Bu.T)`` over many rows in one launch (weights ``(N, K)``)."""
    kinds = {"silu": 1, "gelu_tanh": 2}
    if activation not in kinds:
        raise ValueError(f"gemm_gated_pair: activation {activation!r} is neither 'silu' nor 'gelu_tanh'")
    _numel(_dev(A, "A"), M * K, "A")
    _numel(_dev(Bg, "Bg"), N * K, "Bg")
    _numel(_dev(Bu, "Bu"), N * K, "Bu")
    _numel(_dev(G, "G"), M * N, "G")
    _numel(_dev(C, "C"), M * N, "C")
    check(lib().iron_gemm_gated_pair_bf16(ptr(A), ptr(Bg), ptr(Bu), ptr(G), ptr(C), M, N, K, kinds[activation],
                                          ptr(_word(valid, "valid")), current_stream()), "iron_gemm_gated_pair_bf16")


def gemv_fused(W, x, y, *, M, K, W2=None, norm_w=None, eps=0.0, residual=None, residual_scale=1.0, epilogue=0):
    """One-row fusion: ``[RMSNorm ->] GEMV [-> + residual | gate/up -> SiLU -> Mul]``."""
    _numel(_dev(W, "W"), M * K, "W")
    _numel(_dev(x, "x"), K, "x")
    _numel(_dev(y, "y"), M, "y")
    if W2 is not None:
        _numel(_dev(W2, "W2"), M * K, "W2")
    if norm_w is not None:
        _numel(_dev(norm_w, "norm_w"), K, "norm_w")
    if residual is not None:
        _numel(_dev(residual, "residual"), M, "residual")
    check(
        lib().iron_gemv_fused_bf16(ptr(W), ptr(W2), ptr(x), ptr(norm_w), float(eps), ptr(residual),
                                   float(residual_scale), ptr(y), M, K, int(epilogue), current_stream()),
        "iron_gemv_fused_bf16",
    )


def decode_qkv(x, norm_w, Wq, Wk, Wv, angles, q_out, keys, values, *, eps, hidden, heads, kv_heads, d,
               cache_rows, position, angle_row=None, table=None, token=None):
    """Attention's first half for one token: norm, q/k/v projections, RoPE, cache writes.  ``angles``
    is the token's row of the RoPE table, or with ``angle_row`` (a device word) the whole table.  With
    ``table`` and ``token`` (a device word) the input is that row of the embedding table, which the
    launch also writes to ``x``."""
    _numel(_dev(x, "x"), hidden, "x")
    _numel(_dev(norm_w, "norm_w"), hidden, "norm_w")
    _numel(_dev(Wq, "Wq"), heads * d * hidden, "Wq")
    _numel(_dev(Wk, "Wk"), kv_heads * d * hidden, "Wk")
    _numel(_dev(Wv, "Wv"), kv_heads * d * hidden, "Wv")
    _dev(angles, "angles")
    if angle_row is None:
        _numel(angles, d, "angles")
    elif angles.numel() % d or angles.numel() < d:
        raise ValueError(f"angles: a table of rows of {d}, got {angles.numel()} elements")
    _numel(_dev(q_out, "q_out"), heads * d, "q_out")
    _numel(_dev(keys, "keys"), cache_rows * kv_heads * d, "keys")
    _numel(_dev(values, "values"), cache_rows * kv_heads * d, "values")
    if table is not None:
        _dev(table, "table")
        if table.numel() % hidden or table.numel() < hidden:
            raise ValueError(f"table: rows of {hidden}, got {table.numel()} elements")
        check(
            lib().iron_decode_qkv_embed_bf16(ptr(table), ptr(_word(token, "token")), table.numel() // hidden, ptr(x),
                                             ptr(norm_w), float(eps), ptr(Wq), ptr(Wk), ptr(Wv), ptr(angles),
                                             ptr(q_out), ptr(keys), ptr(values), hidden, heads, kv_heads, d, cache_rows,
                                             ptr(_word(position, "position")), ptr(_word(angle_row, "angle_row")),
                                             angles.numel() // d, current_stream()),
            "iron_decode_qkv_embed_bf16",
        )
        return
    check(
        lib().iron_decode_qkv_bf16(ptr(x), ptr(norm_w), float(eps), ptr(Wq), ptr(Wk), ptr(Wv), ptr(angles),
                                   ptr(q_out), ptr(keys), ptr(values), hidden, heads, kv_heads, d, cache_rows,
                                   ptr(_word(position, "position")), ptr(_word(angle_row, "angle_row")),
                                   angles.numel() // d, current_stream()),
        "iron_decode_qkv_bf16",
    )


def decode_heads(q, q_out, *, heads, kv_heads, d, eps, norms=0, k=None, v=None, q_gain=None, k_gain=None,
                 q_angles=None, k_angles=None, rotary=0, two_halves=True, keys=None, values=None, row0=None,
                 row1=None, cache_rows=0):
    """Per-head norms, RoPE and the cache rows of one token's q, k, v (``iron_decode_heads_bf16``)."""
    _numel(_dev(q, "q"), heads * d, "q")
    _numel(_dev(q_out, "q_out"), heads * d, "q_out")
    for name, t, n in (("k", k, kv_heads * d), ("v", v, kv_heads * d), ("q_gain", q_gain, d), ("k_gain", k_gain, d),
                       ("q_angles", q_angles, rotary), ("k_angles", k_angles, rotary),
                       ("keys", keys, cache_rows * kv_heads * d), ("values", values, cache_rows * kv_heads * d)):
        if t is not None:
            _numel(_dev(t, name), n, name)
    check(
        lib().iron_decode_heads_bf16(ptr(q), ptr(k), ptr(v), ptr(q_gain), ptr(k_gain), int(norms), float(eps),
                                     ptr(q_angles), ptr(k_angles), int(rotary), int(two_halves), ptr(q_out), ptr(keys),
                                     ptr(values), ptr(_word(row0, "row0")), ptr(_word(row1, "row1")), int(cache_rows),
                                     heads, kv_heads, d, current_stream()),
        "iron_decode_heads_bf16",
    )


def prefill_qkv(x, Wq, Wk, Wv, angles, q_out, k_out, v_out, *, rows, hidden, heads, kv_heads, d, valid=None):
    """A prompt chunk's q/k/v projections with q and k turned by RoPE, one launch."""
    _numel(_dev(x, "x"), rows * hidden, "x")
    _numel(_dev(Wq, "Wq"), heads * d * hidden, "Wq")
    _numel(_dev(Wk, "Wk"), kv_heads * d * hidden, "Wk")
    _numel(_dev(Wv, "Wv"), kv_heads * d * hidden, "Wv")
    _numel(_dev(angles, "angles"), rows * d, "angles")
    _numel(_dev(q_out, "q_out"), rows * heads * d, "q_out")
    _numel(_dev(k_out, "k_out"), rows * kv_heads * d, "k_out")
    _numel(_dev(v_out, "v_out"), rows * kv_heads * d, "v_out")
    check(
        lib().iron_prefill_qkv_bf16(ptr(x), ptr(Wq), ptr(Wk), ptr(Wv), ptr(angles), ptr(q_out), ptr(k_out),
                                    ptr(v_out), rows, hidden, heads, kv_heads, d, ptr(_word(valid, "valid")),
                                    current_stream()),
        "iron_prefill_qkv_bf16",
    )


def prefill_qkv_cache(x, Wq, Wk, Wv, angles, q_out, keys, values, *, rows, hidden, heads, kv_heads, d, cache_rows,
                      start, valid=None):
    """``prefill_qkv`` with k and v written into rows ``start`` on of the layer's KV caches."""
    _numel(_dev(x, "x"), rows * hidden, "x")
    _numel(_dev(Wq, "Wq"), heads * d * hidden, "Wq")
    _numel(_dev(Wk, "Wk"), kv_heads * d * hidden, "Wk")
    _numel(_dev(Wv, "Wv"), kv_heads * d * hidden, "Wv")
    _numel(_dev(angles, "angles"), rows * d, "angles")
    _numel(_dev(q_out, "q_out"), rows * heads * d, "q_out")
    _numel(_dev(keys, "keys"), cache_rows * kv_heads * d, "keys")
    _numel(_dev(values, "values"), cache_rows * kv_heads * d, "values")
    check(
        lib().iron_prefill_qkv_cache_bf16(ptr(x), ptr(Wq), ptr(Wk), ptr(Wv), ptr(angles), ptr(q_out), ptr(keys),
                                          ptr(values), rows, hidden, heads, kv_heads, d, cache_rows,
                                          ptr(_word(start, "start")), ptr(_word(valid, "valid")), current_stream()),
        "iron_prefill_qkv_cache_bf16",
    )


def rmsnorm(x, w, y, *, rows, cols, eps, valid=None, residual=None):
    """``residual``: the normed rows are added to it (the sum rounded as the separate step rounds)."""
    _numel(_dev(x, "x"), rows * cols, "x")
    _numel(_dev(y, "y"), rows * cols, "y")
    if w is not None:
        _numel(_dev(w, "weight"), cols, "weight")
    if residual is not None:
        _numel(_dev(residual, "residual"), rows * cols, "residual")
        check(
            lib().iron_rmsnorm_add_bf16(ptr(x), ptr(w), ptr(residual), ptr(y), rows, cols, float(eps),
                                        ptr(_word(valid, "valid")), current_stream()),
            "iron_rmsnorm_add_bf16",
        )
        return
    check(
        lib().iron_rmsnorm_bf16(
            ptr(x), ptr(w), ptr(y), rows, cols, float(eps), ptr(_word(valid, "valid")),
            current_stream(),
        ),
        "iron_rmsnorm_bf16",
    )


def rope(x, angles, y, *, rows, cols, angle_rows, two_halves=True, valid=None, row_cols=None):
    """``cols`` columns of each row turn; ``row_cols`` (default: the same) is the whole row, whose
    remaining columns pass through."""
    row_cols = cols if row_cols is None else row_cols
    _numel(_dev(x, "x"), rows * row_cols, "x")
    _numel(_dev(angles, "angles"), angle_rows * cols, "angles")
    _numel(_dev(y, "y"), rows * row_cols, "y")
    if row_cols == cols:
        check(lib().iron_rope_bf16(ptr(x), ptr(angles), ptr(y), rows, cols, angle_rows, int(two_halves),
                                   ptr(_word(valid, "valid")), current_stream()), "iron_rope_bf16")
    else:
        check(lib().iron_rope_partial_bf16(ptr(x), ptr(angles), ptr(y), rows, row_cols, cols, angle_rows,
                                           int(two_halves), ptr(_word(valid, "valid")), current_stream()),
              "iron_rope_partial_bf16")


def _binary(name):
    def call(a, b, y, *, n=None, valid=None):
        n = y.numel() if n is None else n
        _numel(_dev(a, "a"), n, "a")
        _numel(_dev(b, "b"), n, "b")
        _numel(_dev(y, "y"), n, "y")
        check(
            getattr(lib(), name)(ptr(a), ptr(b), ptr(y), n, ptr(_word(valid, "valid")), current_stream()),
            name,
        )

    call.__name__ = name
    return call


mul = _binary("iron_mul_bf16")
add = _binary("iron_add_bf16")
silu_mul = _binary("iron_silu_mul_bf16")


def row_broadcast(x, row, y, *, rows, cols, multiply=False, valid=None):
    """``y[r] = x[r] + row`` (or ``* row``) for every row ``r`` under the bound."""
    _numel(_dev(x, "x"), rows * cols, "x")
    _numel(_dev(row, "row"), cols, "row")
    _numel(_dev(y, "y"), rows * cols, "y")
    check(
        lib().iron_row_broadcast_bf16(ptr(x), ptr(row), ptr(y), rows, cols, int(bool(multiply)),
                                      ptr(_word(valid, "valid")), current_stream()),
        "iron_row_broadcast_bf16",
    )


def silu(x, y, *, n=None, valid=None):
    n = y.numel() if n is None else n
    _numel(_dev(x, "x"), n, "x")
    _numel(_dev(y, "y"), n, "y")
    check(lib().iron_silu_bf16(ptr(x), ptr(y), n, ptr(_word(valid, "valid")), current_stream()), "iron_silu_bf16")


UNARY = {"gelu_tanh": 0, "gelu_erf": 1, "relu": 2, "sigmoid": 3, "tanh": 4, "clamp": 5}


def unary(x, y, kind, *, n=None, low=0.0, high=0.0, valid=None):
    """``y = f(x)``, ``kind`` one of ``UNARY``; ``low`` and ``high`` are the clamp's bounds."""
    n = y.numel() if n is None else n
    _numel(_dev(x, "x"), n, "x")
    _numel(_dev(y, "y"), n, "y")
    check(lib().iron_unary_bf16(ptr(x), ptr(y), n, UNARY[kind], float(low), float(high), ptr(_word(valid, "valid")),
                                current_stream()), "iron_unary_bf16")


def axpy(x, y, out, *, a, n=None, valid=None):
    n = out.numel() if n is None else n
    _numel(_dev(x, "x"), n, "x")
    _numel(_dev(y, "y"), n, "y")
    _numel(_dev(out, "out"), n, "out")
    check(lib().iron_axpy_bf16(ptr(x), ptr(y), ptr(out), n, float(a), ptr(_word(valid, "valid")), current_stream()),
          "iron_axpy_bf16")


def layernorm(x, w, y, *, rows, cols, eps, valid=None):
    _numel(_dev(x, "x"), rows * cols, "x")
    _numel(_dev(y, "y"), rows * cols, "y")
    if w is not None:
        _numel(_dev(w, "weight"), cols, "weight")
    check(lib().iron_layernorm_bf16(ptr(x), ptr(w), ptr(y), rows, cols, float(eps), ptr(_word(valid, "valid")),
                                    current_stream()), "iron_layernorm_bf16")


def softmax(x, y, *, rows, cols, addend=None, soft_cap=None, length=None):
    """Softmax of each row of ``x`` (bf16 or float32) over its first ``length`` columns (a device word)."""
    f32 = x.dtype == torch.float32
    _numel(_dev(x, "x", torch.float32 if f32 else torch.bfloat16), rows * cols, "x")
    _numel(_dev(y, "y"), rows * cols, "y")
    if addend is not None:
        _numel(_dev(addend, "addend", torch.float32), rows * cols, "addend")
    check(lib().iron_softmax_bf16(ptr(x), int(f32), ptr(addend), ptr(y), rows, cols, float(soft_cap or 0.0),
                                  ptr(_word(length, "length")), current_stream()), "iron_softmax_bf16")


def mha_prefill(
    Q, K, V, O, *, heads, kv_heads, d, seq, seq_len=None, kv_len, scale=None, causal=True,
    window=None, q_interleaved=False, kv_interleaved=False, valid=None, kv_valid=None, kv_first=None, kv_rows=None,
):
    """``kv_first`` (a device word) and ``kv_rows``: K and V are buffers of ``kv_rows`` rows (at the
    least; ``kv_interleaved``) of which the ``kv_len`` from row ``*kv_first`` on are the keys."""
    seq_len = seq if seq_len is None else seq_len
    scale = 1.0 / math.sqrt(d) if scale is None else scale
    _numel(_dev(Q, "Q"), seq * heads * d, "Q")
    _numel(_dev(O, "O"), seq * heads * d, "O")
    if kv_first is not None:
        _window(K, V, kv_rows, kv_len, kv_heads, d, kv_interleaved)
        check(
            lib().iron_mha_prefill_at_bf16(
                ptr(Q), ptr(K), ptr(V), ptr(O), heads, kv_heads, d, seq, seq_len, kv_len, float(scale),
                int(causal), -1 if window is None else int(window), int(q_interleaved),
                ptr(_word(valid, "valid")), ptr(_word(kv_valid, "kv_valid")), ptr(_word(kv_first, "kv_first")),
                int(kv_rows), current_stream(),
            ),
            "iron_mha_prefill_at_bf16",
        )
        return
    _numel(_dev(K, "K"), kv_len * kv_heads * d, "K")
    _numel(_dev(V, "V"), kv_len * kv_heads * d, "V")
    check(
        lib().iron_mha_prefill_bf16(
            ptr(Q), ptr(K), ptr(V), ptr(O), heads, kv_heads, d, seq, seq_len, kv_len, float(scale),
            int(causal), -1 if window is None else int(window), int(q_interleaved),
            int(kv_interleaved), ptr(_word(valid, "valid")), ptr(_word(kv_valid, "kv_valid")),
            current_stream(),
        ),
        "iron_mha_prefill_bf16",
    )


def _window(K, V, kv_rows, kv_len, kv_heads, d, kv_interleaved):
    if not kv_interleaved or kv_rows is None or kv_rows < kv_len:
        raise ValueError(f"a window of the keys takes them row by row (kv_interleaved) out of kv_rows ({kv_rows}) "
                         f">= kv_len ({kv_len})")
    for name, t in (("K", K), ("V", V)):
        if _dev(t, name).numel() < kv_rows * kv_heads * d:
            raise ValueError(f"{name}: expected {kv_rows * kv_heads * d} elements at the least, got {t.numel()}")


def mha_decode_workspace(heads, d, device="cuda"):
    n = lib().iron_mha_decode_workspace_bytes(heads, d)
    return torch.empty(n // 4, dtype=torch.float32, device=device)


def mha_decode(
    Q, K, V, O, *, heads, kv_heads, d, kv_len, scale=None, window=None, kv_interleaved=False,
    kv_valid=None, workspace, kv_first=None, kv_rows=None, form=0, short_keys=0,
):
    """``kv_first`` / ``kv_rows``: the keys are a window of a longer buffer, as ``mha_prefill``'s.
    ``form`` / ``short_keys`` force the kernel form (``iron_mha_decode_tuned_bf16``)."""
    scale = 1.0 / math.sqrt(d) if scale is None else scale
    _numel(_dev(Q, "Q"), heads * d, "Q")
    _numel(_dev(O, "O"), heads * d, "O")
    _dev(workspace, "workspace", torch.float32)
    need = lib().iron_mha_decode_workspace_bytes(heads, d)
    if workspace.numel() * 4 < need:
        raise ValueError(f"workspace: {workspace.numel() * 4} bytes, need {need}")
    if kv_first is not None:
        _window(K, V, kv_rows, kv_len, kv_heads, d, kv_interleaved)
        check(
            lib().iron_mha_decode_at_bf16(
                ptr(Q), ptr(K), ptr(V), ptr(O), heads, kv_heads, d, kv_len, float(scale),
                -1 if window is None else int(window), ptr(_word(kv_valid, "kv_valid")),
                ptr(_word(kv_first, "kv_first")), int(kv_rows), ptr(workspace), current_stream(),
            ),
            "iron_mha_decode_at_bf16",
        )
        return
    _numel(_dev(K, "K"), kv_len * kv_heads * d, "K")
    _numel(_dev(V, "V"), kv_len * kv_heads * d, "V")
    if form or short_keys:
        check(
            lib().iron_mha_decode_tuned_bf16(
                ptr(Q), ptr(K), ptr(V), ptr(O), heads, kv_heads, d, kv_len, float(scale),
                -1 if window is None else int(window), int(kv_interleaved),
                ptr(_word(kv_valid, "kv_valid")), ptr(workspace), int(form), int(short_keys), current_stream(),
            ),
            "iron_mha_decode_tuned_bf16",
        )
        return
    check(
        lib().iron_mha_decode_bf16(
            ptr(Q), ptr(K), ptr(V), ptr(O), heads, kv_heads, d, kv_len, float(scale),
            -1 if window is None else int(window), int(kv_interleaved),
            ptr(_word(kv_valid, "kv_valid")), ptr(workspace), current_stream(),
        ),
        "iron_mha_decode_bf16",
    )


def mha_decode_static(Q, K, V, O, *, heads, kv_heads, d, kv_len, scale=None, window=None, kv_interleaved=False,
                      kv_valid=None):
    """``mha_decode`` with the split-KV partial results in the library's own device scratch: no
    workspace, nothing allocated (for callers that cannot allocate); refused past its fixed size."""
    scale = 1.0 / math.sqrt(d) if scale is None else scale
    _numel(_dev(Q, "Q"), heads * d, "Q")
    _numel(_dev(O, "O"), heads * d, "O")
    _numel(_dev(K, "K"), kv_len * kv_heads * d, "K")
    _numel(_dev(V, "V"), kv_len * kv_heads * d, "V")
    check(
        lib().iron_mha_decode_static_bf16(
            ptr(Q), ptr(K), ptr(V), ptr(O), heads, kv_heads, d, kv_len, float(scale),
            -1 if window is None else int(window), int(kv_interleaved),
            ptr(_word(kv_valid, "kv_valid")), current_stream(),
        ),
        "iron_mha_decode_static_bf16",
    )


def gather_rows(table, ids, out, *, valid=None):
    _dev(table, "table", None)
    _dev(ids, "ids", torch.int32)
    _dev(out, "out", table.dtype)
    row_bytes = table[0].numel() * table.element_size()
    n_ids = ids.numel()
    _numel(out, n_ids * table[0].numel(), "out")
    check(
        lib().iron_gather_rows(
            ptr(table), ptr(ids), ptr(out), n_ids, table.shape[0], row_bytes,
            ptr(_word(valid, "valid")), current_stream(),
        ),
        "iron_gather_rows",
    )


def copy_rows(src, dst, *, rows, row_elems, src_rows, dst_rows, src_stride=None, dst_stride=None,
              src_row=None, dst_row=None, valid=None):
    """``dst[dst_row + i] = src[src_row + i]`` for ``i < rows``; strides in elements."""
    _dev(src, "src", None)
    _dev(dst, "dst", src.dtype)
    es = src.element_size()
    src_stride = row_elems if src_stride is None else src_stride
    dst_stride = row_elems if dst_stride is None else dst_stride
    if src.numel() < (src_rows - 1) * src_stride + row_elems:
        raise ValueError(f"src: {src.numel()} elements do not hold {src_rows} rows")
    if dst.numel() < (dst_rows - 1) * dst_stride + row_elems:
        raise ValueError(f"dst: {dst.numel()} elements do not hold {dst_rows} rows")
    check(
        lib().iron_copy_rows(
            ptr(src), ptr(dst), rows, row_elems * es, src_stride * es, dst_stride * es, src_rows,
            dst_rows, ptr(_word(src_row, "src_row")), ptr(_word(dst_row, "dst_row")),
            ptr(_word(valid, "valid")), current_stream(),
        ),
        "iron_copy_rows",
    )


def argmax(logits, token, *, n=None, record=None, at=None, token_copy=None):
    n = logits.numel() if n is None else n
    _dev(logits, "logits")
    _dev(token, "token", torch.int32)
    if record is not None:
        _dev(record, "record", torch.int32)
    check(
        lib().iron_argmax_bf16(
            ptr(logits), n, ptr(token), ptr(record), 0 if record is None else record.numel(),
            ptr(_word(at, "at")), ptr(_word(token_copy, "token_copy")), current_stream(),
        ),
        "iron_argmax_bf16",
    )


def sample_workspace(n, device="cuda"):
    """The draw's workspace, zeroed: its first words count a launch's blocks and start at zero."""
    return torch.zeros(lib().iron_sample_workspace_bytes(n) // 8, dtype=torch.int64, device=device)


def sample(logits, draws, token, *, n=None, row=None, k_max=64, workspace=None, record=None, at=None,
           token_copy=None, advance=None):
    """The draw of ``draws``' row at word ``row`` (a device word, or None for the first row).
    ``advance``: ``(words, exprs, n)`` -- word expressions the same launch evaluates once the token is
    written (``eval_words``'s, for the tail of a replayed decode step)."""
    n = logits.numel() if n is None else n
    _dev(logits, "logits")
    _dev(token, "token", torch.int32)
    if draws is not None:
        _dev(draws, "draws", torch.int32)
    if record is not None:
        _dev(record, "record", torch.int32)
    if workspace is None:
        workspace = sample_workspace(n, logits.device)
    need = lib().iron_sample_workspace_bytes(n)
    if workspace.numel() * workspace.element_size() < need:
        raise ValueError(f"workspace: {workspace.numel() * workspace.element_size()} bytes, need {need}")
    common = (ptr(logits), n, ptr(draws), 0 if draws is None else draws.numel(), ptr(_word(row, "row")), k_max,
              ptr(workspace), ptr(token), ptr(record), 0 if record is None else record.numel(),
              ptr(_word(at, "at")), ptr(_word(token_copy, "token_copy")))
    if advance is None:
        check(lib().iron_sample_bf16(*common, current_stream()), "iron_sample_bf16")
        return
    words, exprs, count = advance
    _dev(words, "words", torch.int32)
    _dev(exprs, "exprs", torch.int32)
    if exprs.numel() < 9 * count:
        raise ValueError(f"exprs: {exprs.numel()} words hold fewer than {count} expressions of 9")
    check(lib().iron_sample_advance_bf16(*common, ptr(words), words.numel(), ptr(exprs), count, current_stream()),
          "iron_sample_advance_bf16")


def eval_words(words, exprs, n=None):
    _dev(words, "words", torch.int32)
    _dev(exprs, "exprs", torch.int32)
    n = exprs.numel() // 9 if n is None else n  # nine words a record
    check(lib().iron_eval_words(ptr(words), words.numel(), ptr(exprs), n, current_stream()), "iron_eval_words")


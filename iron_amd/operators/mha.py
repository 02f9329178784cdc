"""MHA: fused attention, grouped-query, causal / windowed, the queries the keys' last rows.

The reference's operator (iron/operators/mha.py:191-1239).  Many queries run the MFMA
flash kernel ``iron_mha_prefill_bf16``; one query (``seq_len == 1``, the reference's
"packed" decode) runs the split-KV streaming kernel ``iron_mha_decode_bf16``.  Per-call
``valid`` bounds the queries and ``kv_valid`` the keys, so the work follows the context,
not the cache.
"""

from __future__ import annotations

import numpy as np

from ..common.declare import Built, In, Operator, Out, Scratch, Select, ceildiv, param, per_call, tunable
from ..common.testing import Case, Testing
from ..common.verify import Tolerance

# One query: up to this many live keys one launch does it all (a block a query head); a cache that can
# hold more takes the launch whose blocks choose by the live keys, and a merge launch behind it.
SHORT_KEYS = 2048

_CASES = [
    Case(dict(num_heads=1, seq_len=16384), bench=True),
    Case(dict(num_heads=8, num_KV_heads=2, seq_len=16384), extensive=True, bench=True),
    # A chunk over a cache: 2048 queries, the last rows of 8192 keys.
    Case(dict(num_heads=8, num_KV_heads=2, seq_len=2048, kv_len=8192)),
    # One query over a cache: Llama 3.2 1B's decode.
    Case(dict(num_heads=32, num_KV_heads=8, seq_len=1, kv_len=2048, heads_interleaved=True)),
    Case(dict(num_heads=40, num_KV_heads=8, d=64, seq_len=1, kv_len=2048, heads_interleaved=True)),
    Case(dict(num_heads=24, num_KV_heads=8, d=128, seq_len=1, kv_len=2048, heads_interleaved=True)),
    Case(dict(num_heads=8, num_KV_heads=2, seq_len=1, kv_len=512), extensive=True),
    Case(dict(num_heads=8, num_KV_heads=2, seq_len=2048, d=128), extensive=True),
    # Llama 3.2 1B's prefill.
    Case(dict(num_heads=32, num_KV_heads=8, seq_len=2048, heads_interleaved=True, kv_interleaved=True), bench=True),
]


class MHA(Operator):
    test = Testing(_CASES)

    num_heads: int = param()
    num_KV_heads: int = param(default=lambda op: op.num_heads)
    seq_len: int = param(default=lambda op: op.seq_pad)
    # The block Q's rows are whole of: 64 as on the reference's device; a graph whose rows
    # are not whole blocks records 1 (the HIP kernels need no padding).
    seq_unit: int = param(default=64, repr=False)
    seq_pad: int = param(derive=lambda op: op.seq_padding(op.seq_len), repr=False)
    # A cache longer than the queries, whose last rows the queries are.
    kv_len: int = param(default=lambda op: op.seq_pad)
    # ``(seq, heads, d)`` as a projection writes it, so no copy reorders the heads.
    heads_interleaved: bool = param(default=False)
    kv_interleaved: bool = param(default=False)
    d: int = param(default=64)
    causal: bool = param(default=True, array=True)
    # Keys more than this many positions from a query are masked.
    window: int | None = param(default=None, array=True)
    scale: float = param(default=lambda op: float(1 / np.sqrt(op.d)), array=True)
    # One query: the split-KV kernel.
    packed: bool = param(derive=lambda op: op.seq_len == 1, repr=False, array=True, init=False)
    # The reference's AIE tunables: accepted, carried, not used by the HIP launch.
    B_q: int = tunable()
    num_pipelines: int = tunable(default=1)
    pv_cores: int = tunable(repr=False)
    workspace_words: int = param(derive=lambda op: op._workspace_words(), repr=False)

    Q = In(Select(heads_interleaved, (seq_pad, num_heads, d), (num_heads, seq_pad, d)))
    K = In(Select(kv_interleaved, (kv_len, num_KV_heads, d), (num_KV_heads, kv_len, d)))
    V = In(Select(kv_interleaved, (kv_len, num_KV_heads, d), (num_KV_heads, kv_len, d)))
    O = Out(Select(heads_interleaved, (seq_pad, num_heads, d), (num_heads, seq_pad, d)))  # noqa: E741
    # Split-KV partial results of the one-query kernel.
    workspace = Scratch(workspace_words, dtype=np.float32, when=packed)
    # A bound on the queries limits the compute; a bound on the keys limits K's and V's rows.
    valid = per_call(bounds=seq_pad)
    kv_valid = per_call(bounds=kv_len)

    def _workspace_words(self) -> int:
        if self.seq_len != 1:
            return 0
        from .._lib import lib

        return int(lib().iron_mha_decode_workspace_bytes(self.num_heads, self.d)) // 4

    def seq_padding(self, seq_len: int) -> int:
        """``seq_len`` rounded up to ``seq_unit``; one query is not padded (mha.py:516-520)."""
        if seq_len == 1:
            return 1
        return ceildiv(seq_len, self.seq_unit) * self.seq_unit

    @property
    def q_tokens(self) -> int:
        return self.valid if "_extents" in vars(self) and "valid" in vars(self)["_extents"] else self.seq_len

    @property
    def kv_tokens(self) -> int:
        ext = vars(self).get("_extents", {})
        if "kv_valid" in ext:
            return ext["kv_valid"]
        return self.kv_len - self.seq_pad + self.q_tokens

    def validate(self) -> None:
        if self.d not in (64, 128, 256, 512):
            raise ValueError(f"MHA: d ({self.d}) must be 64, 128, 256 or 512")
        if self.window is not None and self.window <= 0:
            raise ValueError(f"MHA: window ({self.window}) must be positive or None")
        if not 0 <= self.scale < np.inf:
            raise ValueError(f"MHA: scale ({self.scale}) must be finite and not negative")
        if self.num_heads <= 0:
            raise ValueError(f"MHA: num_heads ({self.num_heads}) must be at least 1")
        if self.num_KV_heads <= 0:
            raise ValueError(f"MHA: num_KV_heads ({self.num_KV_heads}) must be at least 1")
        if self.num_KV_heads > self.num_heads:
            raise ValueError(f"MHA: num_KV_heads ({self.num_KV_heads}) must be at most num_heads ({self.num_heads})")
        if self.num_heads % self.num_KV_heads:
            raise ValueError(f"MHA: num_heads ({self.num_heads}) must be a multiple of "
                             f"num_KV_heads ({self.num_KV_heads})")
        if self.seq_len <= 0:
            raise ValueError(f"MHA: seq_len ({self.seq_len}) must be at least 1")
        if self.kv_len < self.seq_pad:
            raise ValueError(f"MHA: kv_len ({self.kv_len}) must be at least seq_pad ({self.seq_pad}): "
                             "the queries are its last rows")
        group = self.num_heads // self.num_KV_heads
        if self.seq_len == 1 and group not in (1, 2, 3, 4, 5, 6, 8) and not (
                group <= 16 and (self.d in (64, 128) or self.kv_len <= SHORT_KEYS)) and self.d != 512:
            raise ValueError(f"MHA: one query takes up to 16 query heads per KV head at d = 64 or 128 "
                             f"(1, 2, 3, 4, 5, 6 or 8 at d = 256 over more than {SHORT_KEYS} keys), not {group}")
        if self.seq_len == 1 and not self.causal and self.window is not None:
            raise ValueError("MHA: one query past every key attends backwards: causal")

    @classmethod
    def infer(cls, shapes, heads_interleaved=False, kv_interleaved=False, **kw):
        q, k = shapes["Q"], shapes["K"]
        if len(q) != 3 or len(k) != 3:
            raise ValueError(f"Q {q} and K {k} are (seq, heads, d) or (heads, seq, d)")
        seq, heads = (q[0], q[1]) if heads_interleaved else (q[1], q[0])
        kv_len, kv_heads = (k[0], k[1]) if kv_interleaved else (k[1], k[0])
        out = dict(num_heads=heads, num_KV_heads=kv_heads, seq_len=seq, kv_len=kv_len, d=q[2])
        if seq != 1 and seq % 64:
            out["seq_unit"] = 1
        return out

    def bind_views(self, inputs, outputs):
        bound = {}
        q, k = inputs.get("Q"), inputs.get("K")
        if q is not None and 0 in q.valid:
            if not self.heads_interleaved:
                raise ValueError("MHA: a bound on the queries needs heads_interleaved (seq on the first axis)")
            bound["valid"] = q.valid[0]
        if k is not None and 0 in k.valid:
            if not self.kv_interleaved:
                raise ValueError("MHA: a bound on the keys needs kv_interleaved (keys on the first axis)")
            bound["kv_valid"] = k.valid[0]
        return bound

    def takes_view(self, name: str) -> bool:
        """K and V may be a window of a longer buffer whose first row a call names (a ring cache's)."""
        return name in ("K", "V") and self.kv_interleaved

    def output_valid(self, name, inputs):
        q = inputs.get("Q")
        return {0: q.valid[0]} if name == "O" and q is not None and 0 in q.valid else {}

    def ops(self) -> int:
        """Q K^T and its product with V per head, over the keys each query keeps (mha.py:1064-1071)."""
        keys = self.kv_len - self.seq_pad + self.seq_len
        position = keys - self.seq_len + np.arange(self.seq_len)
        ahead = 0 if self.causal else (self.window or keys)
        lo = np.maximum(position - self.window, 0) if self.window else 0
        hi = np.minimum(position + ahead, keys - 1)
        return 4 * self.num_heads * self.d * int((hi - lo + 1).sum())

    def tolerance(self) -> Tolerance:
        return Tolerance(rtol=0.04, atol=0.15, max_mismatch_frac=0.005,
                         note="the reference's (mha.py:1118-1126); measured within rtol 1e-2 / atol 1e-2")

    def build(self) -> Built:
        from .. import kernels

        H, G, d, L = self.num_heads, self.num_KV_heads, self.d, self.kv_len
        scale, window = float(self.scale), self.window
        if self.packed:
            kvi = self.kv_interleaved
            own = {}

            # While the context stays within SHORT_KEYS rows, attention over the cache's first
            # SHORT_KEYS rows is the same attention, in one launch: a graph that follows its per-call
            # values on the host captures that form too and replays it for as long as it holds.
            bounded = ("kv_valid", SHORT_KEYS) if kvi and L > SHORT_KEYS and d != 512 else None

            def launch(t, words):
                ws = t.get("workspace")
                if ws is None:  # a call outside a graph: allocated once, kept
                    ws = own.get("ws")
                    if ws is None:
                        ws = own["ws"] = kernels.mha_decode_workspace(H, d, t["Q"].device)
                keys, values, rows, ring = t["K"], t["V"], L, _key_window(words, G * d)
                if bounded and not ring and (words.get("__context__") or {}).get("bounded"):
                    rows = SHORT_KEYS
                    keys, values = keys.reshape(-1)[: rows * G * d], values.reshape(-1)[: rows * G * d]
                kernels.mha_decode(t["Q"], keys, values, t["O"], heads=H, kv_heads=G, d=d, kv_len=rows,
                                   scale=scale, window=window, kv_interleaved=kvi,
                                   kv_valid=words.get("kv_valid"), workspace=ws, **ring)

            return Built("iron_mha_decode_bf16", launch, bounded)
        seq, seq_len, causal = self.seq_pad, self.seq_len, self.causal
        qi, kvi = self.heads_interleaved, self.kv_interleaved

        def launch(t, words):
            kernels.mha_prefill(t["Q"], t["K"], t["V"], t["O"], heads=H, kv_heads=G, d=d, seq=seq,
                                seq_len=seq_len, kv_len=L, scale=scale, causal=causal, window=window,
                                q_interleaved=qi, kv_interleaved=kvi, valid=words.get("valid"),
                                kv_valid=words.get("kv_valid"), **_key_window(words, G * d))

        return Built("iron_mha_prefill_bf16", launch)


def _key_window(words, row: int) -> dict:
    """The launch's ``kv_first`` / ``kv_rows`` where K and V are windows of a longer buffer: both from
    the same first row, a row of the buffer ``row`` elements."""
    views = words.get("__views__") or {}
    k, v = views.get("K"), views.get("V")
    if k is None and v is None:
        return {}
    if k is None or v is None or k["index"] is None or v["index"] is None or k["ids"] is not None or v["ids"] is not None:
        if all(x is None or (x["index"] is None and x["ids"] is None) for x in (k, v)):
            return {}   # bounded only
        raise ValueError("MHA: K and V are windows of their buffers from the same row, or neither is")
    if k["index"].data_ptr() != v["index"].data_ptr() or k["rows"] != v["rows"] or k["stride"] != row or v["stride"] != row:
        raise ValueError("MHA: K's and V's windows start at the same row of buffers alike")
    return dict(kv_first=k["index"], kv_rows=k["rows"])

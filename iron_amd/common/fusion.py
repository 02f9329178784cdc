"""Step fusion for the versions of a graph.

The recorded steps stay what the reference records -- one operator per step, which is
what ``Graph.reference`` and check mode run.  When a version is loaded for the GPU, runs
of single-row steps that a decoder layer always records together are launched as one
fused kernel each (``iron_amd/csrc/fused.hip``), which rounds wherever the separate steps
round:

  RMSNorm, GEMV q/k/v, RoPE q/k, Copy k/v -> cache      => iron_decode_qkv_bf16
  RMSNorm, GEMV gate, GEMV up, SiLU, ElementwiseMul      => iron_gemv_fused_bf16 (epilogue 2)
  ... with GELU (tanh) for SiLU                          => iron_gemv_fused_bf16 (epilogue 3)
  GEMV, ElementwiseAdd / AXPY (the residual)             => iron_gemv_fused_bf16 (epilogue 1)
  RMSNorm, GEMV (the head; or a layer's q, k, v)         => iron_gemv_fused_bf16 (epilogue 0) each
  GEMV, GELU (tanh) or SiLU, Mul by a given row          => iron_gemv_fused_bf16 (epilogue 4 / 5)
  RMSNorm per head of q/k/v, RoPE q/k, Copy k/v -> cache => iron_decode_heads_bf16

in a prompt chunk's version (several rows, 64-wide heads),

  GEMM q/k/v (one input), RoPE q/k                       => iron_prefill_qkv_bf16
  ... and Copy k/v -> the chunk's cache rows             => iron_prefill_qkv_cache_bf16
  GEMM (gate), GEMM (up), SiLU or GELU (tanh), Mul       => iron_gemm_gated_pair_bf16
  GEMM (up), SiLU or GELU (tanh) of the gate, Mul        => iron_gemm_gated_bf16
  SiLU, ElementwiseMul (no such product before them)     => iron_silu_mul_bf16
  GEMM, ElementwiseAdd / AXPY (the residual)             => iron_gemm_residual_bf16
  ... few rows over a long K, and the RMSNorm after them => iron_gemm_residual_norm_bf16

and in either,

  RMSNorm, ElementwiseAdd (a sandwich layer's residual)  => iron_rmsnorm_add_bf16

A run is fused only if every intermediate it hides is read by nothing else.
"""

from __future__ import annotations

import dataclasses
from collections import Counter
from collections.abc import Callable
from typing import Any


@dataclasses.dataclass
class Fused:
    """One launch standing for ``steps`` consecutive recorded steps."""

    kind: str
    first: int
    count: int
    launch: Callable[[], None]
    launches: int = 1      # 0: a step other launches made needless (nothing runs for it)
    scratch_bytes: int = 0  # device memory of its own the launch needs, live over the run


class _Anything:
    """Stands for a tensor while runs are only being matched (before the arena is loaded)."""

    def reshape(self, *a):
        return self

    def __getitem__(self, key):
        return self


def match(recording) -> list[Fused]:
    """The runs ``plan`` would fuse, without binding any tensor: for the arena plan, which must
    keep every buffer a run touches alive across the whole run."""
    return plan(recording, lambda h: _Anything(), lambda e: None, lambda first, nbytes: _Anything())


def _plain(h) -> bool:
    return h.index is None and h.ids is None and not h.valid


def _name(step) -> str:
    return type(step.op).__name__


def _same(a, b) -> bool:
    """Two handles that are the same elements of the same buffer."""
    return a.buffer is b.buffer and a.offset == b.offset and a.elements == b.elements and _plain(a) and _plain(b)


def _same_view(a, b) -> bool:
    """The same elements of the same buffer, whatever bound each carries."""
    return (a.buffer is b.buffer and a.offset == b.offset and a.elements == b.elements
            and a.index is None and a.ids is None and b.index is None and b.ids is None)


def plan(recording, tensor: Callable[[Any], Any], word: Callable[[Any], Any],
         scratch: Callable[[int, int], Any] | None = None) -> list[Fused]:
    """The fused launches of ``recording``'s steps, by the first step each covers.

    ``tensor(handle)`` is the device tensor behind a handle, ``word(expr)`` the device word
    of a per-call expression, ``scratch(first, nbytes)`` the device memory placed for the run
    that starts at step ``first`` (``Fused.scratch_bytes`` of it); without ``scratch`` no run
    that needs memory of its own is planned.
    """
    from .. import kernels

    steps = recording.steps
    reads: Counter = Counter()
    for s in steps:
        for h in s.inputs.values():
            reads[id(h.buffer)] += 1
            if h.ids is not None:
                reads[id(h.ids.buffer)] += 1
    for h in recording.outputs:
        reads[id(h.buffer)] += 1
    for v in (recording.carry or {}).values():
        if hasattr(v, "buffer"):
            reads[id(v.buffer)] += 1

    def once(h, n=1) -> bool:
        return h.buffer.kind == "transient" and reads[id(h.buffer)] == n

    def norm_row(s) -> bool:
        return (_name(s) == "RMSNorm" and s.op.rows == 1 and s.op.weighted and not s.values
                and all(_plain(h) for h in (*s.inputs.values(), *s.outputs.values())))

    def gemv_row(s, x=None) -> bool:
        ok = (_name(s) == "GEMV" and s.op.num_batches is None and not s.values
              and all(_plain(h) for h in (*s.inputs.values(), *s.outputs.values())))
        return ok and (x is None or _same(s.inputs["B"], x))

    def gated_at(j, before=None):
        """``(args, kw)`` of ``iron_gemm_gated_bf16`` where steps j, j + 1, j + 2 are a many-row product, the
        activation of an earlier product of the same shape (the gate) and their Mul, or None.  With
        ``before``, the step right ahead of them must be the product that made the gate, of the same
        rows by the same bound and read by the activation alone."""
        if j + 2 >= len(steps):
            return None
        s, sl, ml = steps[j], steps[j + 1], steps[j + 2]
        if not (_name(s) == "GEMM"
                and (_name(sl) == "SiLU" or (_name(sl) == "GELU" and sl.op.approximate == "tanh"))
                and _name(ml) == "ElementwiseMul"
                and s.op.b_col_maj and not s.op.c_col_maj and "valid_k" not in s.values
                and s.op.M >= 64 and s.op.N >= 64 and s.op.K % 64 == 0):
            return None
        up, gate, act = s.outputs["C"], sl.inputs["x"], sl.outputs["y"]
        a, b = ml.inputs["a"], ml.inputs["b"]
        paired = (_same_view(a, act) and _same_view(b, up)) or (_same_view(a, up) and _same_view(b, act))
        gv, sv, mv = s.values.get("valid"), sl.values.get("valid"), ml.values.get("valid")
        # the elementwise bounds count elements, the product's rows
        bounds_agree = sv == mv and ((gv is None and sv is None) or (
            gv is not None and sv is not None and gv.value == sv.value and gv.linear and sv.linear
            and sv.scale == gv.scale * s.op.N and sv.bias == gv.bias * s.op.N))
        flat = all(h.index is None and h.ids is None
                   for h in (*s.inputs.values(), up, gate, act, a, b, ml.outputs["y"]))
        if not (paired and flat and once(up) and once(act) and bounds_agree and gate.buffer is not up.buffer
                and gate.elements == up.elements and sl.op.size == up.elements and ml.op.size == up.elements
                and ml.outputs["y"].elements == up.elements
                and set(sl.values) <= {"valid"} and set(ml.values) <= {"valid"}):
            return None
        if before is not None:
            g = before
            if not (_name(g) == "GEMM" and g.op.b_col_maj and not g.op.c_col_maj and "valid_k" not in g.values
                    and (g.op.M, g.op.N, g.op.K) == (s.op.M, s.op.N, s.op.K) and g.values.get("valid") == gv
                    and _same_view(g.inputs["A"], s.inputs["A"]) and _same_view(g.outputs["C"], gate) and once(gate)
                    and gate.buffer is not ml.outputs["y"].buffer
                    and all(h.index is None and h.ids is None for h in (*g.inputs.values(), g.outputs["C"]))):
                return None
        args = dict(A=tensor(s.inputs["A"]), B=tensor(s.inputs["B"]), G=tensor(gate), C=tensor(ml.outputs["y"]))
        kw = dict(M=s.op.M, N=s.op.N, K=s.op.K, valid=word(gv),
                  activation="silu" if _name(sl) == "SiLU" else "gelu_tanh")
        return args, kw

    def same_data(a, b) -> bool:
        return (a is not None and b is not None and a.buffer is b.buffer and a.offset == b.offset
                and a.elements == b.elements and _plain(a) and _plain(b))

    def heads_finish_at(j):
        """The launch for the steps from ``j`` on where they are what lies between a token's q/k/v
        projections and its attention in a layer that norms its heads one by one: RMSNorm per head of
        q (of k, of v), RoPE on q (and k), k's and v's copies into their cache rows -- or None."""
        first = steps[j]
        # the projections just ahead: q's product is what this norm reads; k's and v's follow it
        back = j
        while back > 0 and j - back < 3 and gemv_row(steps[back - 1]):
            back -= 1
        made = [g.outputs["C"] for g in steps[back:j]]
        at = next((n for n, h in enumerate(made) if same_data(h, first.inputs["x"])), None)
        if at is None or len(made) - at not in (1, 3):
            return None
        cur = {"q": made[at], "k": made[at + 1] if len(made) - at == 3 else None,
               "v": made[at + 2] if len(made) - at == 3 else None}
        d = first.op.tile_size
        if any(h is not None and h.elements % d for h in cur.values()) or d % 16 or d > 2048:
            return None
        heads = cur["q"].elements // d
        kv_heads = cur["k"].elements // d if cur["k"] is not None else 1
        if cur["k"] is not None and cur["v"].elements != cur["k"].elements:
            return None
        p, norms, eps, gains = j, 0, None, {"q": None, "k": None}
        for bit, name in enumerate(("q", "k", "v")):
            st = steps[p] if p < len(steps) else None
            if (cur[name] is None or st is None or _name(st) != "RMSNorm" or st.values or st.op.tile_size != d
                    or not same_data(st.inputs["x"], cur[name]) or not once(cur[name]) or not _plain(st.outputs["y"])
                    or (eps is not None and float(st.op.epsilon) != eps) or (name == "v" and st.op.weighted)):
                continue
            if st.op.weighted:
                if not _plain(st.inputs["weight"]) or st.inputs["weight"].elements != d:
                    return None
                gains[name] = st.inputs["weight"]
            norms |= 1 << bit
            eps = float(st.op.epsilon)
            cur[name] = st.outputs["y"]
            p += 1
        if not norms & 1:
            return None
        angles, rotary, two_halves = {"q": None, "k": None}, 0, True
        for name in ("q", "k"):
            st = steps[p] if p < len(steps) else None
            if (cur[name] is None or st is None or _name(st) != "RoPE" or st.values or st.op.angle_rows != 1
                    or st.op.row != d or st.op.cols % 16 or not same_data(st.inputs["x"], cur[name])
                    or not once(cur[name]) or not _plain(st.inputs["angles"]) or not _plain(st.outputs["y"])
                    or (rotary and (st.op.cols, st.op.two_halves) != (rotary, two_halves))):
                continue
            angles[name], rotary, two_halves = st.inputs["angles"], st.op.cols, bool(st.op.two_halves)
            cur[name] = st.outputs["y"]
            p += 1
        # k's copies into its cache rows (the slot and, in a ring, its mirror), then v's into the same rows
        caches, rows_at = {}, None
        for name in ("k", "v"):
            if cur[name] is None:
                continue
            found = []
            while p < len(steps) and len(found) < 2 and _name(steps[p]) == "Copy" and not steps[p].values:
                cp = steps[p]
                src, dst = cp.inputs["src"], cp.outputs["dst"]
                if not (same_data(src, cur[name]) and dst.index is not None and dst.ids is None and not dst.valid
                        and dst.offset == 0 and dst.index_stride == cur[name].elements
                        and dst.elements == cur[name].elements
                        and (not found or dst.buffer is found[0].buffer)):
                    break
                found.append(dst)
                p += 1
            if not found or not once(cur[name], len(found)):
                return None
            if rows_at is None:
                rows_at = [f.index for f in found]
            elif [f.index for f in found] != rows_at or found[0].index_rows != caches["k"].index_rows:
                return None
            caches[name] = found[0]
        if p - j < 2:
            return None
        args = dict(q=tensor(made[at]).reshape(-1), q_out=tensor(cur["q"]).reshape(-1))
        kw = dict(heads=heads, kv_heads=kv_heads, d=d, eps=eps, norms=norms, rotary=rotary, two_halves=two_halves)
        for name in ("q", "k"):
            if gains[name] is not None:
                args[f"{name}_gain"] = tensor(gains[name]).reshape(-1)
            if angles[name] is not None:
                args[f"{name}_angles"] = tensor(angles[name]).reshape(-1)
        if caches:
            kd, vd = caches["k"], caches["v"]
            args |= dict(k=tensor(made[at + 1]).reshape(-1), v=tensor(made[at + 2]).reshape(-1),
                         keys=tensor(kd)[: kd.index_rows * kd.index_stride],
                         values=tensor(vd)[: vd.index_rows * vd.index_stride])
            kw |= dict(cache_rows=kd.index_rows, row0=word(rows_at[0]),
                       row1=word(rows_at[1]) if len(rows_at) > 1 else None)
        return Fused("decode_heads", j, p - j, lambda a=args, kw=kw: kernels.decode_heads(**a, **kw))

    fused: list[Fused] = []
    # decode_qkv launches whose RoPE row is a copy of one table row: (producing step, args, kw)
    rope_rows: list[tuple[int, dict, dict]] = []
    # decode_qkv launches whose input row is a copy of one row of a table (the token's embedding)
    embed_rows: list[tuple[int, dict, dict]] = []
    i = 0
    while i < len(steps):
        s = steps[i]
        got = None
        if norm_row(s):
            n = s.outputs["y"]
            rest = steps[i + 1 :]
            # attention's first half
            if (len(rest) >= 7 and all(gemv_row(g, n) for g in rest[:3]) and once(n, 3)
                    and _name(rest[3]) == "RoPE" and _name(rest[4]) == "RoPE"
                    and _name(rest[5]) == "Copy" and _name(rest[6]) == "Copy"):
                gq, gk, gv, rq, rk, ck, cv = rest[:7]
                q, k, v = (g.outputs["C"] for g in (gq, gk, gv))
                d = rq.op.cols
                kd, vd = ck.outputs["dst"], cv.outputs["dst"]
                ok = (
                    _same(rq.inputs["x"], q) and _same(rk.inputs["x"], k) and once(q) and once(k) and once(v)
                    and rq.op.two_halves and rk.op.two_halves and rq.op.angle_rows == 1 and rk.op.angle_rows == 1
                    and rq.op.row == rq.op.cols and rk.op.row == rk.op.cols
                    and rk.op.cols == d and d in (64, 128) and not rq.values and not rk.values
                    and rq.inputs["angles"].buffer is rk.inputs["angles"].buffer and _plain(rq.inputs["angles"])
                    and _same(ck.inputs["src"], rk.outputs["y"]) and once(rk.outputs["y"])
                    and _same(cv.inputs["src"], v)
                    and kd.index is not None and vd.index is not None and kd.index == vd.index
                    and kd.ids is None and vd.ids is None and not kd.valid and not vd.valid
                    and kd.offset == 0 and vd.offset == 0
                    and kd.index_stride == k.elements and vd.index_stride == v.elements
                    and k.elements == v.elements and k.elements % d == 0 and q.elements % d == 0
                )
                if ok:
                    args = dict(
                        x=tensor(s.inputs["x"]).reshape(-1), norm_w=tensor(s.inputs["weight"]).reshape(-1),
                        Wq=tensor(gq.inputs["A"]), Wk=tensor(gk.inputs["A"]), Wv=tensor(gv.inputs["A"]),
                        angles=tensor(rq.inputs["angles"]).reshape(-1), q_out=tensor(rq.outputs["y"]).reshape(-1),
                        keys=tensor(kd)[: kd.index_rows * kd.index_stride],
                        values=tensor(vd)[: vd.index_rows * vd.index_stride],
                    )
                    kw = dict(eps=float(s.op.epsilon), hidden=s.op.tile_size, heads=q.elements // d,
                              kv_heads=k.elements // d, d=d, cache_rows=kd.index_rows, position=word(kd.index))
                    got = Fused("decode_qkv", i, 8, lambda a=args, kw=kw: kernels.decode_qkv(**a, **kw))
                    made_by = _row_copy(steps, i, rq.inputs["angles"], d)
                    if made_by is not None:
                        rope_rows.append((made_by, args, kw))
                    # ... and the layer's input where it is one row of an embedding table
                    looked_up = _row_copy(steps, i, s.inputs["x"], s.op.tile_size)
                    if looked_up is not None and not any(
                            h.buffer is s.inputs["x"].buffer for t in steps[looked_up + 1 : i] for h in t.inputs.values()):
                        embed_rows.append((looked_up, args, kw))
            # the gated MLP's first half
            if (got is None and len(rest) >= 4 and gemv_row(rest[0], n) and gemv_row(rest[1], n) and once(n, 2)
                    and (_name(rest[2]) == "SiLU" or (_name(rest[2]) == "GELU" and rest[2].op.approximate == "tanh"))
                    and _name(rest[3]) == "ElementwiseMul"):
                gg, gu, si, mu = rest[:4]
                g, u = gg.outputs["C"], gu.outputs["C"]
                ok = (_same(si.inputs["x"], g) and once(g) and once(u) and once(si.outputs["y"])
                      and not si.values and not mu.values
                      and _same(mu.inputs["a"], si.outputs["y"]) and _same(mu.inputs["b"], u)
                      and gg.op.M == gu.op.M and gg.op.K == gu.op.K and _plain(mu.outputs["y"]))
                if ok:
                    args = dict(W=tensor(gg.inputs["A"]), W2=tensor(gu.inputs["A"]),
                                x=tensor(s.inputs["x"]).reshape(-1), norm_w=tensor(s.inputs["weight"]).reshape(-1),
                                y=tensor(mu.outputs["y"]).reshape(-1))
                    kw = dict(M=gg.op.M, K=gg.op.K, eps=float(s.op.epsilon), epilogue=2 if _name(si) == "SiLU" else 3)
                    got = Fused("norm_gate_up_silu_mul" if _name(si) == "SiLU" else "norm_gate_up_gelu_mul", i, 5, lambda a=args, kw=kw: kernels.gemv_fused(**a, **kw))
            # the head: norm, then one projection -- or a layer's q, k, v projections where something
            # other than RoPE follows them (heads normed one by one): the norm rides each one's prologue
            if got is None:
                count = 0
                while count < 3 and count < len(rest) and gemv_row(rest[count], n):
                    count += 1
                if count and once(n, count):
                    calls = []
                    for g0 in rest[:count]:
                        args = dict(W=tensor(g0.inputs["A"]), x=tensor(s.inputs["x"]).reshape(-1),
                                    norm_w=tensor(s.inputs["weight"]).reshape(-1), y=tensor(g0.outputs["C"]).reshape(-1))
                        calls.append((args, dict(M=g0.op.M, K=g0.op.K, eps=float(s.op.epsilon), epilogue=0)))

                    def norm_gemvs(calls=calls):
                        for a, kw in calls:
                            kernels.gemv_fused(**a, **kw)

                    got = Fused("norm_gemv", i, 1 + count, norm_gemvs, launches=count)
        elif (_name(s) == "GEMM" and len(steps) - i >= 5
              and [_name(t) for t in steps[i + 1 : i + 5]] == ["GEMM", "GEMM", "RoPE", "RoPE"]):
            # a prompt chunk's projections and rotations
            gq, gk, gv, rq, rk = steps[i : i + 5]
            a = gq.inputs["A"]

            def rows_gemm(g):
                return (g.op.b_col_maj and not g.op.c_col_maj and "valid_k" not in g.values
                        and _same_view(g.inputs["A"], a) and g.op.M == gq.op.M and g.op.K == gq.op.K
                        and all(h.index is None and h.ids is None for h in (*g.inputs.values(), *g.outputs.values())))

            q, k, v = (g.outputs["C"] for g in (gq, gk, gv))
            M, d = gq.op.M, 64
            ok = (
                all(rows_gemm(g) for g in (gq, gk, gv)) and once(q) and once(k)
                and M >= 64 and gq.op.K % 64 == 0 and gq.op.N % 128 == 0 and gk.op.N % 128 == 0
                and gk.op.N == gv.op.N
                and _same_view(rq.inputs["x"], q) and _same_view(rk.inputs["x"], k)
                and all(r.op.two_halves and r.op.cols == d and r.op.row == d and r.op.angle_rows == M for r in (rq, rk))
                and rq.op.rows * d == M * gq.op.N and rk.op.rows * d == M * gk.op.N
                and rq.inputs["angles"].buffer is rk.inputs["angles"].buffer
                and _same_view(rq.inputs["angles"], rk.inputs["angles"])
                and all(h.index is None and h.ids is None for h in (rq.outputs["y"], rk.outputs["y"]))
            )
            if ok:
                args = dict(x=tensor(a), Wq=tensor(gq.inputs["B"]), Wk=tensor(gk.inputs["B"]), Wv=tensor(gv.inputs["B"]),
                            angles=tensor(rq.inputs["angles"]), q_out=tensor(rq.outputs["y"]),
                            k_out=tensor(rk.outputs["y"]), v_out=tensor(v))
                kw = dict(rows=M, hidden=gq.op.K, heads=gq.op.N // d, kv_heads=gk.op.N // d, d=d,
                          valid=word(gq.values.get("valid")))
                got = Fused("prefill_qkv", i, 5, lambda a=args, kw=kw: kernels.prefill_qkv(**a, **kw))
                # ... and the two copies of k and v into the chunk's rows of the layer's caches
                ck, cv = (steps[i + 5], steps[i + 6]) if i + 6 < len(steps) else (None, None)
                if ck is not None and _name(ck) == "Copy" and _name(cv) == "Copy":
                    kd, vd = ck.outputs["dst"], cv.outputs["dst"]
                    gvalid = gq.values.get("valid")
                    cached = (
                        _same_view(ck.inputs["src"], rk.outputs["y"]) and _same_view(cv.inputs["src"], v)
                        and once(rk.outputs["y"]) and once(v)
                        and all(h.index is not None and h.ids is None and h.offset == 0
                                and h.index_stride == gk.op.N and h.elements == M * gk.op.N for h in (kd, vd))
                        and kd.index == vd.index and kd.index_rows == vd.index_rows
                        and kd.valid.get(0) == gvalid and vd.valid.get(0) == gvalid
                        and ck.inputs["src"].valid.get(0) == gvalid and cv.inputs["src"].valid.get(0) == gvalid
                        and M <= kd.index_rows
                    )
                    if cached:
                        args = {k_: t for k_, t in args.items() if k_ not in ("k_out", "v_out")}
                        args |= dict(keys=tensor(kd)[: kd.index_rows * kd.index_stride],
                                     values=tensor(vd)[: vd.index_rows * vd.index_stride])
                        kw = dict(kw, cache_rows=kd.index_rows, start=word(kd.index))
                        got = Fused("prefill_qkv_cache", i, 7,
                                    lambda a=args, kw=kw: kernels.prefill_qkv_cache(**a, **kw))
        elif (_name(s) == "GEMM" and i + 1 < len(steps) and _name(steps[i + 1]) in ("ElementwiseAdd", "AXPY")
              and s.op.b_col_maj and not s.op.c_col_maj and "valid_k" not in s.values
              and s.op.M >= 64 and s.op.N >= 64 and s.op.K % 64 == 0):
            # a projection over many rows and its residual: the sum rides the product's epilogue
            ad = steps[i + 1]
            c = s.outputs["C"]
            a, b = ad.inputs["a"], ad.inputs["b"]
            if _name(ad) == "AXPY":   # scalar_factor * a + b: the product is the one scaled
                other, scale = (b if _same_view(a, c) else None), float(ad.op.scalar_factor)
            else:
                other, scale = (a if _same_view(b, c) else (b if _same_view(a, c) else None)), 1.0
            gv, av = s.values.get("valid"), ad.values.get("valid")
            # the sum's bound counts elements, the product's rows
            bounds_agree = (gv is None and av is None) or (
                gv is not None and av is not None and gv.value == av.value and gv.linear and av.linear
                and av.scale == gv.scale * s.op.N and av.bias == gv.bias * s.op.N)
            flat = all(h.index is None and h.ids is None
                       for h in (*s.inputs.values(), c, a, b, ad.outputs["y"]))
            if (other is not None and flat and once(c) and bounds_agree and other.elements == c.elements
                    and ad.outputs["y"].elements == c.elements and set(ad.values) <= {"valid"}):
                args = dict(A=tensor(s.inputs["A"]), B=tensor(s.inputs["B"]), R=tensor(other), C=tensor(ad.outputs["y"]))
                kw = dict(M=s.op.M, N=s.op.N, K=s.op.K, residual_scale=scale, valid=word(gv))
                got = Fused("gemm_add", i, 2, lambda a=args, kw=kw: kernels.gemm_residual(**a, **kw))
                # ... and the norm of the rows it leaves (the next layer's input norm after a down
                # projection): few rows over a long K are dealt over several blocks a tile, and the
                # launch that adds their sums up stands where the norm's stood
                nm = steps[i + 2] if i + 2 < len(steps) else None
                need = kernels.gemm_residual_norm_workspace_bytes(s.op.M, s.op.N, s.op.K) if scratch and nm else 0
                if (need and _name(nm) == "RMSNorm" and nm.op.weighted and nm.op.rows == s.op.M
                        and nm.op.tile_size == s.op.N and set(nm.values) <= {"valid"} and nm.values.get("valid") == gv
                        and _same_view(nm.inputs["x"], ad.outputs["y"])
                        and all(h.index is None and h.ids is None for h in (*nm.inputs.values(), nm.outputs["y"]))
                        and nm.outputs["y"].buffer is not ad.outputs["y"].buffer
                        and nm.outputs["y"].buffer is not other.buffer):
                    args = dict(args, gain=tensor(nm.inputs["weight"]), Y=tensor(nm.outputs["y"]),
                                workspace=scratch(i, need))
                    kw = dict(kw, eps=float(nm.op.epsilon))
                    got = Fused("gemm_add_norm", i, 3, lambda a=args, kw=kw: kernels.gemm_residual_norm(**a, **kw),
                                launches=2, scratch_bytes=need)
        elif _name(s) == "GEMM" and (gated := gated_at(i + 1, s)) is not None:
            # a gated feed-forward's two first projections over many rows: one launch computes both
            # products tile by tile, the activated gate riding the second one's epilogue
            args, kw = gated
            args = dict(A=args["A"], Bg=tensor(s.inputs["B"]), Bu=args["B"], G=args["G"], C=args["C"])
            got = Fused("gemm_gated_pair", i, 4, lambda a=args, kw=kw: kernels.gemm_gated_pair(**a, **kw))
        elif _name(s) == "GEMM" and (gated := gated_at(i)) is not None:
            # a gated feed-forward's second projection over many rows: the activated gate rides its epilogue
            args, kw = gated
            got = Fused("gemm_gated", i, 3, lambda a=args, kw=kw: kernels.gemm_gated(**a, **kw))
        elif _name(s) == "SiLU" and i + 1 < len(steps) and _name(steps[i + 1]) == "ElementwiseMul":
            # a gated feed-forward's activation and gate over many rows: one pass instead of two
            m = steps[i + 1]
            act = s.outputs["y"]
            a, b = m.inputs["a"], m.inputs["b"]
            other = b if _same_view(a, act) else (a if _same_view(b, act) else None)
            flat = all(h.index is None and h.ids is None for h in (s.inputs["x"], act, a, b, m.outputs["y"]))
            if (other is not None and flat and once(act) and s.op.size == m.op.size
                    and s.values.get("valid") == m.values.get("valid") and other.elements == act.elements):
                args = dict(a=tensor(s.inputs["x"]).reshape(-1), b=tensor(other).reshape(-1),
                            y=tensor(m.outputs["y"]).reshape(-1))
                kw = dict(n=s.op.size, valid=word(m.values.get("valid")))
                got = Fused("silu_mul", i, 2, lambda a=args, kw=kw: kernels.silu_mul(**a, **kw))
        elif (gemv_row(s) and i + 2 < len(steps) and _name(steps[i + 2]) in ("RowwiseMul", "ElementwiseMul")
              and (_name(steps[i + 1]) == "SiLU"
                   or (_name(steps[i + 1]) == "GELU" and steps[i + 1].op.approximate == "tanh"))):
            # a projection, its activation and the product with a given row (a per-layer input's gate)
            ac, mu = steps[i + 1], steps[i + 2]
            c, act = s.outputs["C"], ac.outputs["y"]
            if _name(mu) == "RowwiseMul":   # one row of x by the row: the same product element by element
                a, b = mu.inputs["x"], mu.inputs["row"]
                other = None if mu.op.rows != 1 else (b if same_data(a, act) else (a if same_data(b, act) else None))
            else:
                a, b = mu.inputs["a"], mu.inputs["b"]
                other = b if same_data(a, act) else (a if same_data(b, act) else None)
            if (other is not None and same_data(ac.inputs["x"], c) and once(c) and once(act) and not ac.values
                    and not mu.values and _plain(other) and other.elements == c.elements and _plain(mu.outputs["y"])
                    and mu.outputs["y"].elements == c.elements and other.buffer is not act.buffer):
                args = dict(W=tensor(s.inputs["A"]), x=tensor(s.inputs["B"]).reshape(-1),
                            residual=tensor(other).reshape(-1), y=tensor(mu.outputs["y"]).reshape(-1))
                kw = dict(M=s.op.M, K=s.op.K, epilogue=5 if _name(ac) == "SiLU" else 4)
                got = Fused("gemv_act_mul", i, 3, lambda a=args, kw=kw: kernels.gemv_fused(**a, **kw))
        elif gemv_row(s) and i + 1 < len(steps) and _name(steps[i + 1]) in ("ElementwiseAdd", "AXPY"):
            ad = steps[i + 1]
            c = s.outputs["C"]
            a, b = ad.inputs["a"], ad.inputs["b"]
            if _name(ad) == "AXPY":   # scalar_factor * a + b: the GEMV's row is the one scaled
                other, scale = (b if _same(a, c) else None), float(ad.op.scalar_factor)
            else:
                other, scale = (a if _same(b, c) else (b if _same(a, c) else None)), 1.0
            if other is not None and once(c) and _plain(other) and not ad.values and _plain(ad.outputs["y"]) \
                    and other.elements == c.elements:
                args = dict(W=tensor(s.inputs["A"]), x=tensor(s.inputs["B"]).reshape(-1),
                            residual=tensor(other).reshape(-1), y=tensor(ad.outputs["y"]).reshape(-1))
                kw = dict(M=s.op.M, K=s.op.K, epilogue=1, residual_scale=scale)
                got = Fused("gemv_add", i, 2, lambda a=args, kw=kw: kernels.gemv_fused(**a, **kw))
        if got is None and _name(s) == "RMSNorm" and s.op.rows >= 1 and not s.values:
            got = heads_finish_at(i)
        if (got is None and _name(s) == "RMSNorm" and i + 1 < len(steps) and _name(steps[i + 1]) == "ElementwiseAdd"
                and set(s.values) <= {"valid"}):
            # a block's output normed again before its residual (a sandwich layer): the sum rides the norm's pass
            ad = steps[i + 1]
            n = s.outputs["y"]
            a, b = ad.inputs["a"], ad.inputs["b"]
            other = a if _same_view(b, n) else (b if _same_view(a, n) else None)
            nv, av = s.values.get("valid"), ad.values.get("valid")
            cols = s.op.tile_size
            bounds_agree = (nv is None and av is None) or (
                nv is not None and av is not None and nv.value == av.value and nv.linear and av.linear
                and av.scale == nv.scale * cols and av.bias == nv.bias * cols)
            flat = all(h.index is None and h.ids is None
                       for h in (*s.inputs.values(), n, a, b, ad.outputs["y"]))
            if (other is not None and flat and once(n) and bounds_agree and other.elements == n.elements
                    and ad.outputs["y"].elements == n.elements and set(ad.values) <= {"valid"}):
                args = dict(x=tensor(s.inputs["x"]), w=tensor(s.inputs["weight"]) if s.op.weighted else None,
                            y=tensor(ad.outputs["y"]), residual=tensor(other))
                kw = dict(rows=s.op.rows, cols=cols, eps=float(s.op.epsilon), valid=word(nv))
                got = Fused("norm_add", i, 2, lambda a=args, kw=kw: kernels.rmsnorm(**a, **kw))
        if got is not None:
            fused.append(got)
            i += got.count
        else:
            i += 1
    # A RoPE row copied out of its table for nobody but these launches: they read the table at the
    # call's row themselves, and the copy is not launched.
    for producer in sorted({p for p, _, _ in rope_rows}):
        users = [(a, kw) for p, a, kw in rope_rows if p == producer]
        row = steps[producer].outputs["dst"]
        if reads[id(row.buffer)] != 2 * len(users) or any(f.first <= producer < f.first + f.count for f in fused):
            continue
        table = steps[producer].inputs["src"]
        for a, kw in users:
            a["angles"] = tensor(table).reshape(-1)[: table.index_rows * table.index_stride]
            kw["angle_row"] = word(table.index)
        fused.append(Fused("elided_rope_row", producer, 1, lambda: None, launches=0))
    # The token's embedding row, copied out of its table for a first layer whose fused projections can
    # read the table at the token themselves (and leave the copy where the residual sum reads it).
    for producer, a, kw in embed_rows:
        if any(f.first <= producer < f.first + f.count for f in fused):
            continue
        table = steps[producer].inputs["src"]
        a["table"] = tensor(table).reshape(-1)[: table.index_rows * table.index_stride]
        kw["token"] = word(table.index)
        fused.append(Fused("elided_embedding_row", producer, 1, lambda: None, launches=0))
    return sorted(fused, key=lambda f: f.first)


def _row_copy(steps, before: int, row, width: int):
    """The step before ``before`` that made ``row`` by copying one table row a per-call word names
    (``Copy(table[position])``), or None."""
    for j in range(before - 1, -1, -1):
        s = steps[j]
        if any(h.buffer is row.buffer for h in s.outputs.values()):
            if _name(s) != "Copy":
                return None
            src, dst = s.inputs["src"], s.outputs["dst"]
            ok = (_same(dst, row) and src.index is not None and src.ids is None and not src.valid and src.offset == 0
                  and src.index_stride == width and src.elements == width and src.buffer.kind == "resident"
                  and not s.values)
            return j if ok else None
    return None

"""The decoder's memory modules, device-free: windows, rings, restarts and per-layer RoPE tables
(iron/tests/lm/test_modules.py:216-300), on the toy Llama through the host stand-in."""

import dataclasses

import numpy as np
import pytest

import oracle
from iron_amd.applications.llama import Llama
from iron_amd.lm.blocks import Attention, KVCache, Rope
from iron_amd.lm.causal import OnHost
from tests.llama_support import SCALED, weights

oracle.install()


class HostLlama(OnHost, Llama):
    pass


def small(cls=Llama, **changes):
    config = dataclasses.replace(SCALED, **changes)
    return cls(config, weights(config))


def names(recording):
    return [type(s.op).__name__ for s in recording.steps]


def test_attention_refuses_a_norm_of_other_than_q_k_and_v():
    with pytest.raises(ValueError, match="'qo' names other than q, k and v"):
        Attention(SCALED, 0, norms="qo")


def test_a_cache_attends_within_its_window():
    """Each layer's cache attends within the config's ``sliding_window``, the query's own position
    not counted; one built with no window attends to every position before the query."""
    model = small(sliding_window=65)
    model.layers[1].cache = KVCache(model.config)
    t = model.record(**model.shapes()[1])
    assert [s.op.window for s in t.steps if type(s.op).__name__ == "MHA"] == [64, None]


def test_a_ring_restarts_at_the_chunk_while_it_holds_the_window_before():
    """A ring of 128 positions, a window of 7 and a chunk of 64: positions from 70 on changed after
    70 or 185 ran restart at 64, whose window from 57 the ring still holds, and after 186 at the first."""
    cache = KVCache(dataclasses.replace(SCALED, prefill_chunk=64, max_seq_len=512), 7)
    assert cache.ring == 128 and cache.keys.shape[0] == 256
    assert [cache.restart(70, ran) for ran in (70, 185, 186)] == [64, 64, 0]


def test_a_window_keeps_every_position_where_a_ring_takes_as_many_rows():
    """A ring and its staging take three rings' rows: at a context of three rings or fewer the cache
    keeps every position, at any chunk, a short context's whole one among them."""
    for L, C in ((384, 64), (200, 200)):
        cache = KVCache(dataclasses.replace(SCALED, prefill_chunk=C, max_seq_len=L), 7)
        assert cache.ring is None and cache.keys.shape[0] == L
    with pytest.raises(ValueError, match="no power of two"):
        KVCache(dataclasses.replace(SCALED, prefill_chunk=48, max_seq_len=4096), 7)


def test_a_ring_s_rows_are_per_call_words_of_the_position():
    """A decode step over a ring writes the new row and its mirror and copies the window out; every
    row is a word derived from ``position`` on the device (remainders by the ring, clamps)."""
    model = small(sliding_window=8, max_seq_len=4096, prefill_chunk=64)
    assert model.layers[0].cache.ring == 128 and len(model.recurrent) == 2
    t = model.record()
    values = {"token": 5, "position": 300}
    full = t.check_values(values)
    found = {e.name: e.evaluate(full) for s in t.steps for h in (*s.inputs.values(), *s.outputs.values())
             for e in (h.index, h.valid.get(0)) if e is not None and e.value == "position"}
    assert found["position_r128"] == 300 % 128 and found["position_r128_p128"] == 300 % 128 + 128
    assert found["position_m7_c0__r128"] == (300 - 7) % 128 and found["position_p1_c_8"] == 8
    # Attention reads the window where it lies: K and V are views from the same derived row, and a
    # layer copies only the new row and its mirror, for k and for v.
    mha = [s for s in t.steps if type(s.op).__name__ == "MHA"]
    assert len(mha) == 2 and all(s.inputs["K"].index == s.inputs["V"].index for s in mha)
    assert mha[0].inputs["K"].index.name == "position_m7_c0__r128" and mha[0].inputs["K"].index_rows == 256
    assert names(t).count("Copy") == 2 + 2 * 4


def test_a_ring_s_chunk_attends_from_its_valid_rows_alone():
    """A chunk's queries over a ring are its whole chunk, the rows past ``rows`` masked; the output is
    bounded to ``rows`` again, so ``o_proj`` runs on them alone."""
    model = small(sliding_window=8, max_seq_len=4096)
    assert model.layers[0].cache.ring == 512
    t = model.record(**model.shapes()[1])
    mha = names(t).index("MHA")
    assert not t.steps[mha].inputs["Q"].valid and "valid" not in t.steps[mha].values
    o_proj = next(s for s in t.steps[mha + 1 :] if type(s.op).__name__ == "GEMM")
    assert o_proj.values["valid"].name == "rows"


def test_a_turn_over_a_ring_is_the_run_from_scratch_bit_for_bit():
    """A turn of 150 tokens after 550 ran, over a ring of 512 positions and chunks of 256, reruns its
    chunk from 512; its logits are those of the whole run from scratch."""
    model = small(HostLlama, sliding_window=65, max_seq_len=4096)
    model.load_versions()
    assert model.layers[0].cache.ring == 512
    rng = np.random.default_rng(1)
    whole, other = rng.integers(0, model.config.vocab_size, (2, 700))
    model.logits(whole[:550])
    assert model.session.resume(550) == 512
    turn = model.logits(whole)
    model.logits(other)
    scratch = model.logits(whole)
    np.testing.assert_array_equal(turn, scratch)


def test_a_ring_gives_the_logits_of_the_whole_cache():
    """The same weights and window with the whole cache kept (a context of three rings or fewer)
    and with a ring: the same logits after a prompt of several chunks and after decode steps."""
    kept = small(HostLlama, sliding_window=20, prefill_chunk=64, max_seq_len=256)
    ring = small(HostLlama, sliding_window=20, prefill_chunk=64, max_seq_len=1024)
    assert kept.layers[0].cache.ring is None and ring.layers[0].cache.ring == 128
    kept.load_versions()
    ring.load_versions()
    tokens = np.random.default_rng(2).integers(0, SCALED.vocab_size, 250)
    for n in (40, 200, 201, 202, 250):
        # The same keys in another buffer of another length: the sums' order differs, not the keys.
        a, b = ring.logits(tokens[:n]), kept.logits(tokens[:n])
        assert np.abs(a - b).max() <= 0.02 * np.abs(b).max() and a.argmax() == b.argmax(), n


def test_each_layer_reads_the_rows_of_its_own_rope():
    """A layer holding another ``Rope`` turns q and k by its table's rows, copied once a call however
    many layers hold it; one holding none turns nothing."""
    model = small(num_hidden_layers=3, rope_scaling=None)
    other = Rope(dataclasses.replace(model.config, rope_theta=1e4))
    model.layers[1].rope = model.layers[2].rope = other
    t = model.record(**model.shapes()[1])
    tables = {id(h.buffer.source) for s in t.steps for h in s.inputs.values() if h.buffer.kind == "resident"}
    assert {id(model.rotary_emb.table), id(other.table)} <= tables
    assert names(t).count("RoPE") == 6
    model.layers[0].rope = None
    t = model.record(**model.shapes()[1])
    tables = {id(h.buffer.source) for s in t.steps for h in s.inputs.values() if h.buffer.kind == "resident"}
    assert id(model.rotary_emb.table) not in tables and names(t).count("RoPE") == 4


def test_per_call_expressions_fold_floor_clamp_remainder_and_a_trailing_sum():
    """What a ring's rows are made of: ``clamp(position - W, 0) % R + R`` is one expression of one
    value, evaluated alike on the host and by the device's table (its nine-word record)."""
    from iron_amd.common.graph import Affine, clamp

    p = Affine("position")
    row = clamp(p - 7, lo=0) % 128
    assert [row.evaluate({"position": v}) for v in (0, 7, 8, 135, 300)] == [0, 0, 1, 0, 37]
    mirror = row + 128
    assert mirror.evaluate({"position": 300}) == 165 and (mirror - row).evaluate({"position": 5}) == 128
    assert mirror.record() == [1, -7, 0, 0, 2**31 - 1, 127, 128]
    assert (p * 12 // 12) == p and (p * 12 + 24) // 12 == p + 2      # an even division folds
    assert ((p + 1) // 4).evaluate({"position": 10}) == 2            # a power of two floors
    with pytest.raises(TypeError, match="power of two"):
        (p + 1) // 3
    with pytest.raises(TypeError, match="power of two"):
        p % 12
    with pytest.raises(TypeError):
        clamp(row, hi=5)          # a clamp after a remainder is not one expression
    with pytest.raises(TypeError):
        row * 2
    assert row.name == "position_m7_c0__r128" and mirror.name == "position_m7_c0__r128_p128"


def test_a_number_meets_a_handle_as_a_constant_row():
    """``x * 0.5`` records one rowwise multiply by a bf16 row of that number, the same tensor
    wherever the number and width recur (iron/common/graph/handle.py:652-661)."""
    from iron_amd.common import graph as iron

    class Halve(iron.Graph):
        def body(self, x):
            return (x * 0.5 + x / 2) * 0.5

    t = Halve().record(x=((4, 64), iron.bfloat16))
    assert names(t) == ["RowwiseMul", "RowwiseMul", "ElementwiseAdd", "RowwiseMul"]
    rows = [s.inputs["row"].buffer.source for s in t.steps if type(s.op).__name__ == "RowwiseMul"]
    assert rows[0] is rows[1] is rows[2] and np.all(np.asarray(rows[0].array) == 0.5)


def test_a_profile_in_the_reference_s_format_fills_the_open_tunables_of_recorded_steps(tmp_path):
    """``profiles/<device>.json`` as the reference writes it: entries by operator name, the most
    specific match wins, an unknown operator or field is refused; the tunables are AIE tile counts
    that the steps carry (iron/common/declare/profile.py:26-158)."""
    import iron_amd
    from iron_amd.operators.gemv import GEMV

    E, Q = SCALED.hidden_size, SCALED.num_attention_heads * SCALED.head_dim   # o_proj is (E, Q)
    file = tmp_path / "npu2.json"
    file.write_text('{"entries": [\n'
                    '  {"operator": "GEMV", "tile_size_input": 4},\n'
                    f'  {{"operator": "GEMV", "M": {E}, "K": {Q}, "tile_size_input": 2, "num_aie_columns": 8}},\n'
                    '  {"operator": "RMSNorm", "weighted": true, "rows": 1, "num_aie_columns": 1}\n]}\n')
    profile = iron_amd.Profile.load(file)
    assert len(profile) == 3
    assert profile.tunables_for(GEMV, dict(M=E, K=Q)) == {"tile_size_input": 2, "num_aie_columns": 8}
    assert profile.tunables_for(GEMV, dict(M=64, K=E)) == {"tile_size_input": 4}
    assert profile.make(GEMV, M=E, K=Q, tile_size_input=1).tile_size_input == 1   # what a call gives stays
    model = small()
    model.profile = profile
    t = model.record()
    square = [s.op for s in t.steps if type(s.op).__name__ == "GEMV" and (s.op.M, s.op.K) == (E, Q)]
    assert square and all(op.tile_size_input == 2 and op.num_aie_columns == 8 for op in square)
    assert all(s.op.num_aie_columns == 1 for s in t.steps if type(s.op).__name__ == "RMSNorm" and s.op.weighted)
    again = tmp_path / "again.json"
    profile.save(again)
    assert iron_amd.Profile.load(again).tunables_for(GEMV, dict(M=E, K=Q)) == profile.tunables_for(GEMV, dict(M=E, K=Q))
    file.write_text('{"entries": [{"operator": "Conv2D", "tile": 4}]}')
    with pytest.raises(ValueError, match="no operator 'Conv2D'"):
        iron_amd.Profile.load(file)
    with pytest.raises(TypeError, match="declares no field"):
        profile.add(GEMV, tile_rows=4)
    both = iron_amd.Profile()
    both.add(GEMV, M=E, tile_size_input=2)
    both.add(GEMV, K=Q, tile_size_input=4)
    with pytest.raises(ValueError, match="ambiguous"):
        both.tunables_for(GEMV, dict(M=E, K=Q))


def test_partial_rotary_narrows_the_table_and_turns_the_leading_columns_in_one_step():
    """``rotary_dim``: the angle table is that wide (iron/tests/common/test_decoder.py:51-66), the
    weights keep the whole head, and q and k each take ONE RoPE step over rows a head wide of which
    the leading columns turn (the reference copies them out, rotates and copies back,
    iron/lm/blocks.py:612-620); the step's reference is the rotation of those columns alone."""
    import dataclasses

    import oracle
    from iron_amd.bf16 import round_bf16
    from iron_amd.lm.config import rope_angles
    from oracle import ops

    oracle.install()
    model = small(rotary_dim=32)
    cfg = model.config
    assert cfg.rope_width == 32 and cfg.angles().shape == (cfg.max_seq_len, 32)
    assert np.array_equal(cfg.angles(), rope_angles(32, cfg.max_seq_len, cfg.rope_theta, cfg.rope_scaling))
    assert model.layers[0].self_attn.q_proj.weight.shape == (cfg.num_attention_heads * cfg.head_dim, cfg.hidden_size)
    assert small().config.rotary_dim is None and small().config.rope_width == cfg.head_dim
    for shapes in model.shapes():
        t = model.record(**shapes)
        ropes = [s.op for s in t.steps if type(s.op).__name__ == "RoPE"]
        assert len(ropes) == 2 * cfg.num_hidden_layers
        assert all(op.cols == 32 and op.row == cfg.head_dim for op in ropes)
    op = ropes[0]
    rng = np.random.default_rng(0)
    x = round_bf16(rng.standard_normal((op.rows, op.row)).astype(np.float32))
    table = round_bf16(rope_angles(32, op.angle_rows, cfg.rope_theta))
    got = np.asarray(op.reference(x, table)).reshape(op.rows, op.row)
    assert np.array_equal(got[:, :32], ops.rope(x[:, :32], table)) and np.array_equal(got[:, 32:], x[:, 32:])
    with pytest.raises(ValueError, match="rotary_dim"):
        dataclasses.replace(cfg, rotary_dim=40)

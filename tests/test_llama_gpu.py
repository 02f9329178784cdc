"""The decoder graph on the GPU: compiled versions in one arena, the decode step a HIP graph.

Judged against Hugging Face's float32 logits (the reference's golden fixture) by the
reference's own rule -- within 5 % of the largest logit and the same argmax -- and against
the graph's host reference (the CPU oracle) on the same weights.
"""

import dataclasses

import numpy as np
import pytest

import oracle
from iron_amd.applications.llama import LLAMA_3_2_1B, Llama, shapes
from iron_amd.lm.blocks import KVCache
from iron_amd.lm.causal import OnHost
from oracle import ops
from tests.llama_support import BIASED, BIASED_GOLDEN, SCALED, Golden, assert_close, kl, weights

pytestmark = pytest.mark.gpu
oracle.install()


class HostLlama(OnHost, Llama):
    pass


@pytest.fixture(scope="module")
def golden():
    return Golden()


@pytest.fixture(scope="module")
def toy(cuda):
    model = Llama(SCALED, weights())
    model.load_versions()
    yield model
    model.release()


def test_versions_share_one_arena_and_both_are_hip_graphs(toy):
    decode, prompt = toy.decode_step, toy.prompt_chunk
    assert decode.arena is prompt.arena and decode.arena.buffer is not None
    # the prompt chunk's ids land in its arena slot and its words are rewritten before each replay
    assert decode.captured and prompt.captured
    # 2 + 18 per layer + 3: embed, rope row, the layers, norm, head, draw.
    assert len(decode.recording.steps) == 2 + 18 * SCALED.num_hidden_layers + 3
    names = [type(s.op).__name__ for s in decode.recording.steps]
    assert names.count("GEMV") == 7 * SCALED.num_hidden_layers + 1 and "GEMM" not in names
    pnames = [type(s.op).__name__ for s in prompt.recording.steps]
    assert pnames.count("GEMM") == 7 * SCALED.num_hidden_layers and pnames.count("GEMV") == 1


def test_prompt_then_greedy_decode_matches_hugging_face(toy, golden):
    prompt = np.random.default_rng(7).integers(0, SCALED.vocab_size, 8)
    want = golden.logits(prompt)
    got = toy.logits(prompt)
    assert_close(got, want)
    assert kl(want, got) < 1e-3
    tokens = prompt
    for step in range(6):
        tokens = np.append(tokens, want.argmax())
        want = golden.logits(tokens)
        got = toy.logits(tokens)
        assert_close(got, want, f"step {step}")
        assert kl(want, got) < 1e-3


def test_decode_from_an_empty_cache_token_by_token(toy, golden):
    prompt = np.random.default_rng(7).integers(0, SCALED.vocab_size, 8)
    toy.session.forget(0)
    for n in range(1, len(prompt) + 1):
        last = toy.logits(prompt[:n])
    assert_close(last, golden.logits(prompt))


def test_a_prompt_longer_than_a_chunk_runs_in_chunks(cuda, golden):
    C = SCALED.prefill_chunk
    config = dataclasses.replace(SCALED, max_seq_len=4 * C)
    model = Llama(config, weights())
    model.load_versions()
    tokens = np.random.default_rng(3).integers(0, config.vocab_size, C + 150)
    first = golden.logits(tokens)
    assert_close(model.logits(tokens), first)
    tokens = np.append(tokens, first.argmax())
    assert_close(model.logits(tokens), golden.logits(tokens))
    tokens = np.append(tokens, np.random.default_rng(4).integers(0, config.vocab_size, 30))
    assert_close(model.logits(tokens), golden.logits(tokens))
    model.release()


def test_generate_replays_the_captured_step_and_matches_stepwise_decode(toy):
    """The device-carried run of HIP-graph replays draws the tokens that host-started steps
    draw, and the draw is deterministic."""
    prompt = np.random.default_rng(8).integers(0, SCALED.vocab_size, 40)
    replayed = toy.generate(prompt, 24)
    stepwise = list(toy.session.draw(prompt, 24, each=True))
    again = toy.generate(prompt, 24)
    assert replayed == stepwise == again and len(replayed) == 24
    # ... and the tokens are those the host reference (the oracle) draws.
    host = HostLlama(SCALED, weights())
    host.load_versions()
    assert list(host.session.draw(prompt, 6, each=True)) == replayed[:6]


def test_sampled_tokens_are_the_host_s_token_for_token(toy):
    """Drawn on the device from the sampler's rows (one replayed HIP graph), then drawn again on the
    host from each step's logits at the same seed: the same tokens (iron/lm/testing.py:169-179)."""
    from iron_amd.lm.generation import Sampler, generate_on_host

    prompt = np.random.default_rng(13).integers(0, SCALED.vocab_size, 40)
    drawn = toy.generate(prompt, 24, Sampler(1.5, 50, seed=4))
    assert drawn == list(toy.session.draw(prompt, 24, Sampler(1.5, 50, seed=4), each=True))
    assert drawn == generate_on_host(toy, prompt, 24, Sampler(1.5, 50, seed=4))
    assert drawn != toy.generate(prompt, 24, Sampler(1.5, 50, seed=5))
    # A greedy run after a sampled one finds its rows zero again.
    greedy = toy.generate(prompt, 24)
    assert greedy == generate_on_host(toy, prompt, 24, Sampler(0.0)) and greedy != drawn


def test_a_carried_loop_runs_the_decode_steps_on_the_device(toy):
    """``CarriedLoop(first, body)``: the prompt chunk from the host, then the decode step replayed
    from what each run carried (iron/common/graph/carried.py:189-276); the tokens are generate()'s."""
    import iron_amd

    prompt = np.random.default_rng(8).integers(0, SCALED.vocab_size, 40)
    want = toy.generate(prompt, 24)
    toy.session.forget(0)
    ((ids,), values), = toy.session.chunk_calls(prompt, 0)
    loop = iron_amd.CarriedLoop(toy.prompt_chunk, toy.decode_step)
    assert list(loop.run(23, ids, **values)) == list(range(23))
    record = toy.decode_step.read(toy.drawn)
    assert [int(t) for t in record[len(prompt) - 1 : len(prompt) + 23]] == want
    # The decode step started from the host is a first version too.
    again = iron_amd.CarriedLoop(toy.decode_step, toy.decode_step)
    again.start(token=want[0], position=len(prompt))
    assert len(list(again.steps(5))) == 5
    assert [int(t) for t in toy.decode_step.read(toy.drawn)[len(prompt) : len(prompt) + 6]] == want[1:7]
    with pytest.raises(ValueError, match="takes no tensor"):
        iron_amd.CarriedLoop(toy.decode_step, toy.prompt_chunk)
    with pytest.raises(RuntimeError, match="start"):
        next(iron_amd.CarriedLoop(toy.prompt_chunk, toy.decode_step).steps(1))
    toy.session.forget(0)


def test_replays_past_the_cache_are_refused_before_any_is_launched(toy):
    """A run of replays is checked like a call: the carried position of every step stays inside the
    cache, or none of the run is launched (past a limit the device would drop its writes silently)."""
    L, decode = SCALED.max_seq_len, toy.decode_step
    toy.session.forget(0)
    decode.start(token=1, position=L - 3)
    decode.replay(2)                     # positions L - 2 and L - 1: the cache's last rows
    with pytest.raises(IndexError, match="leave the limits"):
        decode.replay(1)
    decode.start(token=1, position=L - 6)
    with pytest.raises(IndexError, match="leave the limits"):
        decode.replay(6)                 # the sixth would sit at position L
    decode.replay(5)
    toy.session.forget(0)


def test_queued_calls_each_run_on_their_own_per_call_words(cuda):
    """Two calls queued behind long work on the stream, with nothing read back between: the second
    call's words must not replace the first's before the first's copy to the device has run."""
    import torch

    import iron_amd
    from iron_amd.operators import Copy

    class Row(iron_amd.Graph):
        def body(self, table, *, p: iron_amd.Scratchpad[np.int32]):
            row = Copy.step(table[p])
            return row + row

    table = np.arange(64 * 256, dtype=np.float32).reshape(64, 256) % 251
    net = Row().compile(table=(table.shape, iron_amd.bfloat16), capture=False)
    device_table = torch.from_numpy(table).to(torch.bfloat16).cuda()
    net(device_table, p=0)
    torch.cuda.synchronize()
    busy = torch.randn(8192, 8192, device="cuda", dtype=torch.bfloat16)
    for _ in range(30):                  # tens of milliseconds of queued work
        busy @ busy
    first = net(device_table, p=3).tensor.clone()
    second = net(device_table, p=40).tensor.clone()
    torch.cuda.synchronize()
    assert np.array_equal(first.float().cpu().numpy().reshape(-1), 2 * table[3])
    assert np.array_equal(second.float().cpu().numpy().reshape(-1), 2 * table[40])


def test_accuracy_and_determinism_as_the_reference_accepts_a_model(toy):
    """The reference's acceptance of a model on its device (iron/lm/testing.py:136-289): the KL of
    each next-token distribution against the float32 reference's, teacher-forced on the reference's
    greedy tokens, under its bounds (mean 0.02, p90 0.04, max 0.2), and logits bitwise the same run
    after run over two alternating prompts."""
    from iron_amd.lm.generation import accuracy, determinism, kl_stats

    host = HostLlama(SCALED, weights())
    host.load_versions()
    prompt = np.random.default_rng(31).integers(0, SCALED.vocab_size, 24)
    results = accuracy(toy, host, prompt, 10)
    stats = kl_stats(results)
    assert stats["Mean"] < 0.02 and stats["P90"] < 0.04 and stats["Max"] < 0.2, stats
    # The same argmax at every step whose top two the reference holds apart (iron/lm/testing.py:182-206:
    # closer than 5 % of the largest logit, either may win within the logits' own tolerance).
    history = [int(t) for t in prompt]
    for step, (_, same) in enumerate(results):
        want = host.logits(history)
        second, best = np.sort(want)[-2:]
        assert same or best - second <= 0.05 * np.abs(want).max(), f"step {step}: argmax differs on separated logits"
        history.append(int(want.argmax()))
    other = np.random.default_rng(32).integers(0, SCALED.vocab_size, 17)
    assert determinism(toy, [prompt, other], 6, rounds=3) == 0


def test_states_are_read_written_and_pushed(toy):
    """``read`` a state as the device left it, ``push`` what the host wrote into that array,
    ``write`` another (iron/common/graph/compiled.py:840-854); both versions see one arena."""
    prompt = np.random.default_rng(21).integers(0, SCALED.vocab_size, 9)
    toy.logits(prompt)
    decode, chunk, keys = toy.decode_step, toy.prompt_chunk, toy.layers[1].cache.keys
    saved = decode.read(keys).copy()
    assert saved.shape == keys.shape and np.abs(saved[: len(prompt)]).max() > 0
    held = decode.read(keys)
    held[3] = 0.5
    decode.push(keys)
    assert np.array_equal(chunk.read(keys), held) and not np.array_equal(held, saved)
    chunk.write(keys, saved)
    assert np.array_equal(decode.read(keys), saved)
    with pytest.raises(ValueError, match="read the tensor first"):
        chunk.push(toy.layers[0].cache.values)
    decode.upload()
    toy.session.forget(0)


def test_check_mode_judges_every_step_against_its_reference(cuda):
    model = Llama(SCALED, weights())
    model.load_versions(check=True)
    prompt = np.random.default_rng(9).integers(0, SCALED.vocab_size, 12)
    model.logits(prompt)
    model.logits(np.append(prompt, 5))
    model.release()


def test_refusals_before_any_dispatch(toy):
    with pytest.raises(IndexError, match="are outside"):
        toy.logits([1, 2, SCALED.vocab_size])
    with pytest.raises(IndexError):
        toy(token=3, position=SCALED.max_seq_len)  # a position past the cache
    with pytest.raises(TypeError, match="per-call values"):
        toy(token=3, position=0, nonsense=1)
    with pytest.raises(ValueError, match="takes"):
        toy(np.zeros(7, np.int32), token=0, position=0)


@pytest.mark.parametrize("shape", [
    # 128-wide heads (Llama 3 8B's proportions): the prompt chunk's projections stay separate steps
    dict(hidden_size=1024, num_attention_heads=8, num_key_value_heads=2, head_dim=128, intermediate_size=2816),
    # heads that do not come in threes or pairs of tiles, an odd multiple of 64 in the feed-forward, untied head
    dict(hidden_size=768, num_attention_heads=12, num_key_value_heads=4, head_dim=64, intermediate_size=1984,
         tie_word_embeddings=False),
    # one KV head (multi-query), a sliding window shorter than the prompt
    dict(hidden_size=512, num_attention_heads=8, num_key_value_heads=1, head_dim=64, intermediate_size=1024,
         sliding_window=48),
    # a window short enough against the context that the layers keep rings (128 rows, wrapped by the 200-token prompt)
    dict(hidden_size=512, num_attention_heads=8, num_key_value_heads=2, head_dim=64, intermediate_size=1024,
         sliding_window=20, max_seq_len=1024),
    # RoPE over the first half of each head only (partial rotary): one RoPE step turns 32 of 64 columns
    dict(hidden_size=512, num_attention_heads=8, num_key_value_heads=2, head_dim=64, intermediate_size=1024,
         rotary_dim=32),
], ids=["d128", "twelve_heads_untied", "multi_query_window", "ring", "partial_rotary"])
def test_other_decoder_shapes_match_the_host_reference(cuda, shape):
    """Shapes off the benchmark's: every fused path either takes the shape or leaves the steps as
    recorded; either way the GPU's logits are the host reference's, prompt (in two chunks) and decode."""
    config = dataclasses.replace(SCALED, **(dict(vocab_size=1000, num_hidden_layers=2, max_seq_len=256,
                                                 prefill_chunk=64, rope_scaling=None) | shape))
    ring = config.max_seq_len > 256
    assert KVCache(config, config.window).ring == (128 if ring else None)
    names = dict(shapes(config))
    if not config.tie_word_embeddings:
        names["lm_head.weight"] = (config.vocab_size, config.hidden_size)
    w = ops.filled(names, seed=3)
    gpu, cpu = Llama(config, w), HostLlama(config, w)
    gpu.load_versions()
    cpu.load_versions()
    try:
        tokens = np.random.default_rng(5).integers(0, config.vocab_size, 200 if ring else 90)
        want, got = cpu.logits(tokens), gpu.logits(tokens)
        assert_close(got, want)
        for step in range(3):
            tokens = np.append(tokens, want.argmax())
            want, got = cpu.logits(tokens), gpu.logits(tokens)
            assert_close(got, want, f"decode step {step}")
        # The device-carried run draws what host-started steps draw; its first token is the host
        # reference's best within the logits' tolerance (drawn weights leave near-ties).
        drawn = gpu.generate(tokens[:20], 8)
        assert drawn == list(gpu.session.draw(tokens[:20], 8, each=True))
        first = cpu.logits(tokens[:20])
        assert first[drawn[0]] >= first.max() - 0.05 * np.abs(first).max()
    finally:
        gpu.release()


def test_two_layers_at_llama_1b_width_match_the_host_reference(cuda):
    """Llama-3.2-1B's widths (hidden 2048, 32 q / 8 kv heads, intermediate 8192, vocab 128256)
    at two layers: the GPU logits against the graph's host reference on the same weights."""
    config = dataclasses.replace(LLAMA_3_2_1B, num_hidden_layers=2, max_seq_len=512, prefill_chunk=128)
    w = weights(config, seed=1)
    gpu, cpu = Llama(config, w), HostLlama(config, w)
    gpu.load_versions()
    cpu.load_versions()
    tokens = np.random.default_rng(2).integers(0, config.vocab_size, 70)
    want, got = cpu.logits(tokens), gpu.logits(tokens)
    assert_close(got, want)
    tokens = np.append(tokens, want.argmax())
    assert_close(gpu.logits(tokens), cpu.logits(tokens), "decode")
    gpu.release()


def test_a_512_token_prompt_in_a_2048_row_chunk_at_llama_1b_width(cuda):
    """The benchmark's prompt at the benchmark's chunk: 512 tokens under the row bound of a 2048-row
    chunk (the launches whose blocks choose their tiles by the bound), two layers, then a decode
    step, against the host reference on the same weights (whose chunk is as long as the prompt: the
    rows past a bound are nobody's)."""
    config = dataclasses.replace(LLAMA_3_2_1B, num_hidden_layers=2, max_seq_len=2048, prefill_chunk=2048)
    w = weights(config, seed=1)
    gpu, cpu = Llama(config, w), HostLlama(dataclasses.replace(config, prefill_chunk=512), w)
    gpu.load_versions()
    cpu.load_versions()
    try:
        # a layer's down projection, its residual and the next layer's input norm are one run (K dealt
        # over several blocks a tile under this bound, the rows finished and normed by a second launch)
        kinds = [f.kind for f in gpu.prompt_chunk._fused.values()]
        assert kinds.count("gemm_add_norm") == config.num_hidden_layers - 1
        assert kinds.count("gemm_add") == config.num_hidden_layers + 1
        tokens = np.random.default_rng(2).integers(0, config.vocab_size, 512)
        want, got = cpu.logits(tokens), gpu.logits(tokens)
        assert_close(got, want)
        assert kl(want, got) < 0.02
        tokens = np.append(tokens, want.argmax())
        assert_close(gpu.logits(tokens), cpu.logits(tokens), "decode")
    finally:
        gpu.release()


def test_all_sixteen_layers_of_llama_1b_prompt_then_captured_decode(cuda):
    """The benchmark's decoder at its own depth, as the reference accepts a model on its device
    (tests/applications/llama/test.py:63-64 over iron/lm/testing.py:136-206): a 64-token prompt in the
    2048-row chunk, then eight steps of the captured decode graph, teacher-forced on the host
    reference's greedy tokens; each step's logits within 5 % of the largest and the same argmax
    where the top two are apart, the KLs under the reference's bounds."""
    from iron_amd.lm.generation import divergence, greedy, kl_stats

    config = dataclasses.replace(LLAMA_3_2_1B, max_seq_len=2048, prefill_chunk=2048)
    w = weights(config, seed=1)
    gpu, cpu = Llama(config, w), HostLlama(dataclasses.replace(config, prefill_chunk=64), w)
    gpu.load_versions()
    cpu.load_versions()
    try:
        assert gpu.decode_step.captured
        tokens = list(np.random.default_rng(6).integers(0, config.vocab_size, 64))
        results, first = [], None
        for step in range(9):   # the prompt's logits, then eight decode steps
            want, got = cpu.logits(tokens), gpu.logits(tokens)
            assert_close(got, want, f"step {step}")
            results.append(divergence(want, got))
            first = want if first is None else first
            tokens.append(greedy(want))
        stats = kl_stats(results)
        assert stats["Mean"] < 0.02 and stats["P90"] < 0.04 and stats["Max"] < 0.2, stats
        # The device-carried run of replays: its first token is the host reference's best within the
        # logits' tolerance, and the run is the same run after run.
        drawn = gpu.generate(tokens[:64], 8)
        assert first[drawn[0]] >= first.max() - 0.05 * np.abs(first).max()
        assert drawn == gpu.generate(tokens[:64], 8) and len(drawn) == 8
    finally:
        gpu.release()


def _fill_caches(gpu, cpu, n: int, upto: int) -> None:
    """Repeat the caches' first ``n`` rows, a prompt's, up to row ``upto`` -- on the device, and as the
    host model's state (the device's rows, so that what is compared is the step and not the history):
    the reference's ``_fill_caches`` (iron/lm/testing.py:367-392) for linear caches."""
    from iron_amd.common.graph import walk

    version = gpu.decode_step
    device_states = [x for _, x, parent, _ in walk(gpu) if isinstance(parent, KVCache)]
    host_states = [x for _, x, parent, _ in walk(cpu) if isinstance(parent, KVCache)]
    assert device_states and len(device_states) == len(host_states)
    for on_device, on_host in zip(device_states, host_states):
        rows = version.read(on_device)
        for start in range(n, upto, n):
            rows[start : min(start + n, upto)] = rows[: min(n, upto - start)]
        version.push(on_device)
        cpu.decode_step.write(on_host, rows)


@pytest.fixture(scope="module")
def deep(cuda):
    """Two layers at Llama-3.2-1B's width over caches of 16384 rows in 2048-row chunks, on the GPU and
    as the graph's host reference, a 300-token prompt run through both."""
    config = dataclasses.replace(LLAMA_3_2_1B, num_hidden_layers=2, max_seq_len=16384, prefill_chunk=2048)
    w = weights(config, seed=1)
    gpu, cpu = Llama(config, w), HostLlama(dataclasses.replace(config, prefill_chunk=512), w)
    gpu.load_versions()
    cpu.load_versions()
    tokens = np.random.default_rng(21).integers(0, config.vocab_size, 300)
    want, got = cpu.logits(tokens), gpu.logits(tokens)
    assert_close(got, want, "the prompt")
    yield gpu, cpu, tokens, int(want.argmax())
    gpu.release()


@pytest.mark.parametrize("position", [600, 2047, 2048, 5000, 16383])
def test_decode_deep_in_the_cache(deep, position):
    """The reference's ``check_deep_decode`` (iron/lm/testing.py:314-331, held by
    tests/applications/long_context/test.py:215-219): a captured decode step at ``position``, every
    earlier row of the caches filled with the prompt's, against the graph's host reference within
    the reference's KL bound of 0.1 and its 5 % rule.  600 and 2047 replay the graph captured in the
    one-launch form of attention, 2048 on the one whose attention deals the keys over the chip."""
    gpu, cpu, tokens, token = deep
    assert gpu.decode_step.captured and gpu.decode_step._graph_bounded is not None
    _fill_caches(gpu, cpu, len(tokens), position)
    got, _ = gpu(token=token, position=position)
    got = np.array(got.numpy()).ravel()[: gpu.config.vocab_size]
    want, _ = cpu(token=token, position=position)
    want = np.asarray(want.numpy()).ravel()[: gpu.config.vocab_size]
    assert_close(got, want, f"the step at {position}")
    assert kl(want, got) <= 0.1


def test_replays_cross_from_the_bounded_graph_to_the_full_one(deep):
    """A run of device-carried replays that starts under the one-launch form's limit and ends past it
    draws what the same steps draw when each is started from the host."""
    gpu, cpu, tokens, token = deep
    decode = gpu.decode_step
    _fill_caches(gpu, cpu, len(tokens), 2040)
    held = decode.read(gpu.drawn).copy()

    def run(each: bool) -> list[int]:
        _fill_caches(gpu, cpu, len(tokens), 2040)   # the steps wrote rows 2040..: start alike
        decode.start(token=token, position=2040)
        if each:
            for i in range(1, 16):
                drawn = int(decode.read(gpu.drawn)[2040 + i - 1])
                decode.start(token=drawn, position=2040 + i)
        else:
            decode.replay(15)
        return [int(t) for t in decode.read(gpu.drawn)[2040 : 2040 + 16]]

    assert run(each=False) == run(each=True)
    assert held.shape == decode.read(gpu.drawn).shape


def test_prompt_deep_in_the_cache(deep):
    """The reference's ``check_deep_prompt`` (iron/lm/testing.py:334-364): the chunk that holds position
    ``max_seq_len - 1``, 512 rows of it, over caches filled up to the chunk's first row."""
    gpu, cpu, tokens, _ = deep
    C, L = gpu.config.prefill_chunk, gpu.config.max_seq_len
    begin, rows = (L - 1) // C * C, 512
    chunk = np.resize(tokens, rows)
    values = dict(token=int(chunk[-1]), position=begin + rows - 1, start=begin, rows=rows, rope_start=begin)
    _fill_caches(gpu, cpu, len(tokens), begin)
    got, _ = gpu(gpu.session.prompt_ids(chunk), **values)
    got = np.array(got.numpy()).ravel()[: gpu.config.vocab_size]
    want, _ = cpu(cpu.session.prompt_ids(chunk), **values)
    want = np.asarray(want.numpy()).ravel()[: gpu.config.vocab_size]
    assert_close(got, want, f"the chunk at {begin}")
    assert kl(want, got) <= 0.1


def test_a_5000_token_prompt_in_three_chunks_then_replayed_steps(cuda):
    """Toy width, caches of 8192 rows: a prompt of three chunks (attention over a cache longer than
    the chunk), then eight device-carried decode steps past position 5000 (attention's keys dealt
    over the chip, merged by the second launch, inside the captured step), teacher-checked against
    the host model token by token."""
    config = dataclasses.replace(SCALED, max_seq_len=8192, prefill_chunk=2048)
    gpu, cpu = Llama(config, weights()), HostLlama(dataclasses.replace(config, prefill_chunk=1024), weights())
    gpu.load_versions()
    cpu.load_versions()
    try:
        tokens = list(np.random.default_rng(23).integers(0, config.vocab_size, 5000))
        want, got = cpu.logits(tokens), gpu.logits(tokens)
        assert_close(got, want, "the prompt")
        assert kl(want, got) < 1e-2
        drawn = gpu.generate(tokens, 8)
        for step, token in enumerate(drawn):
            want = cpu.logits(tokens)
            assert want[token] >= want.max() - 0.05 * np.abs(want).max(), f"step {step}"
            tokens.append(token)
    finally:
        gpu.release()


def test_fused_decode_step_matches_the_step_by_step_one(cuda, golden):
    """The fused launches compute what the recorded steps compute: same greedy tokens, logits
    within bf16 rounding, and far fewer launches per decode step."""
    fused, plain = Llama(SCALED, weights()), Llama(SCALED, weights())
    fused.load_versions(fuse=True)
    plain.load_versions(fuse=False)
    steps = len(fused.decode_step.recording.steps)
    assert plain.decode_step.launches_per_call == steps
    # per layer 18 steps become 5 launches (qkv, attention, o+add, gate/up, down+add); the head 2 -> 1;
    # neither the RoPE row's copy nor the token's embedding row's is launched (the first layer's
    # projections read both tables at the call's words themselves), and a replay ends with the draw,
    # which evaluates the step's carried and derived words itself.
    assert fused.decode_step.launches_per_call == 5 * SCALED.num_hidden_layers + 2
    assert fused.decode_step.launches_per_replay == fused.decode_step.launches_per_call
    assert plain.decode_step.launches_per_replay == steps
    # the prompt chunk: per layer the three projections, two rotations and two cache writes become
    # one launch, the feed-forward's two first projections, SiLU and Mul another, each residual
    # sum rides its projection's epilogue, and the last row's final norm and head are one
    psteps = len(fused.prompt_chunk.recording.steps)
    assert plain.prompt_chunk.launches_per_call == psteps
    assert fused.prompt_chunk.launches_per_call == psteps - 11 * SCALED.num_hidden_layers - 1
    prompt = np.random.default_rng(7).integers(0, SCALED.vocab_size, 8)
    a, b = fused.logits(prompt), plain.logits(prompt)
    assert np.abs(a - b).max() <= 0.02 * np.abs(b).max()
    long = np.random.default_rng(12).integers(0, SCALED.vocab_size, 200)
    a, b = fused.logits(long), plain.logits(long)
    assert np.abs(a - b).max() <= 0.02 * np.abs(b).max()
    fused.session.forget(0)
    plain.session.forget(0)
    tokens = prompt
    for step in range(6):
        tokens = np.append(tokens, golden.logits(tokens).argmax())
        a, b = fused.logits(tokens), plain.logits(tokens)
        assert np.abs(a - b).max() <= 0.02 * np.abs(b).max(), step
        assert_close(a, golden.logits(tokens), f"fused step {step}")
    # Greedy decoding through the fused step, judged by the step-by-step model on the same context:
    # the two sum in different orders (tile sizes, MFMA shapes), so where the best two logits are
    # closer than that they may pick either; every fused token must be one of the plain model's best.
    prompt = np.random.default_rng(8).integers(0, SCALED.vocab_size, 40)
    drawn = fused.generate(prompt, 24)
    assert len(drawn) == 24
    context = [int(t) for t in prompt]
    for step, token in enumerate(drawn):
        row = plain.logits(np.asarray(context))
        assert row[token] >= row.max() - 0.02 * np.abs(row).max(), (step, token, int(row.argmax()))
        context.append(int(token))
    fused.release()
    plain.release()


def test_fused_kernels_against_the_oracle_at_llama_1b_width(cuda):
    """Each fused kernel through the C ABI against the oracle's steps composed on the host."""
    import torch

    from iron_amd import kernels as K
    from iron_amd.bf16 import from_torch, round_bf16, to_torch
    from oracle import ops

    rng = np.random.default_rng(21)
    E, F, H, G, D, L, pos = 2048, 8192, 32, 8, 64, 64, 37

    def bf(*shape, scale=1.0):
        return round_bf16(rng.standard_normal(shape, dtype=np.float32) * np.float32(scale))

    def dev(a):
        return to_torch(a).to(cuda)

    def close(got, want, atol=2e-2):
        got = (from_torch(got) if isinstance(got, torch.Tensor) else got).reshape(want.shape)
        assert np.all(np.abs(got - want) <= atol + 1e-2 * np.abs(want)), np.abs(got - want).max()

    x, g = bf(E), round_bf16(rng.uniform(0.9, 1.1, E))
    n = ops.rms_norm(x[None], g, epsilon=1e-5)[0]
    # attention's first half
    Wq, Wk, Wv = bf(H * D, E, scale=0.02), bf(G * D, E, scale=0.02), bf(G * D, E, scale=0.02)
    table = round_bf16(ops.rope_angles(D, L))
    keys, values = dev(np.zeros((L, G, D), np.float32)), dev(np.zeros((L, G, D), np.float32))
    q_out = torch.empty(H * D, dtype=torch.bfloat16, device=cuda)
    K.decode_qkv(dev(x), dev(g), dev(Wq), dev(Wk), dev(Wv), dev(table[pos]), q_out, keys, values, eps=1e-5,
                 hidden=E, heads=H, kv_heads=G, d=D, cache_rows=L,
                 position=torch.tensor([pos], dtype=torch.int32, device=cuda))
    close(q_out, ops.rope(ops.gemv(Wq, n).reshape(H, D), table[pos : pos + 1]).reshape(-1))
    # ... and the same launch reading its row out of the whole table by a device word: the same bits
    keys2, values2 = torch.zeros_like(keys), torch.zeros_like(values)
    q2 = torch.empty_like(q_out)
    K.decode_qkv(dev(x), dev(g), dev(Wq), dev(Wk), dev(Wv), dev(table), q2, keys2, values2, eps=1e-5,
                 hidden=E, heads=H, kv_heads=G, d=D, cache_rows=L,
                 position=torch.tensor([pos], dtype=torch.int32, device=cuda),
                 angle_row=torch.tensor([pos], dtype=torch.int32, device=cuda))
    assert torch.equal(q2, q_out) and torch.equal(keys2, keys) and torch.equal(values2, values)
    kc, vc = from_torch(keys), from_torch(values)
    close(kc[pos], ops.rope(ops.gemv(Wk, n).reshape(G, D), table[pos : pos + 1]))
    close(vc[pos], ops.gemv(Wv, n).reshape(G, D))
    assert not kc[:pos].any() and not kc[pos + 1 :].any() and not vc[:pos].any() and not vc[pos + 1 :].any()
    # the gated MLP's first half, and a projection with its residual
    Wg, Wu, Wd = bf(F, E, scale=0.02), bf(F, E, scale=0.02), bf(E, F, scale=0.02)
    m = torch.empty(F, dtype=torch.bfloat16, device=cuda)
    K.gemv_fused(dev(Wg), dev(x), m, M=F, K=E, W2=dev(Wu), norm_w=dev(g), eps=1e-5, epilogue=2)
    want_m = ops.mul(ops.silu(ops.gemv(Wg, n)), ops.gemv(Wu, n))
    close(m, want_m)
    # ... gated by GELU (its tanh form) as Gemma's feed-forward is
    K.gemv_fused(dev(Wg), dev(x), m, M=F, K=E, W2=dev(Wu), norm_w=dev(g), eps=1e-5, epilogue=3)
    close(m, ops.mul(ops.gelu(ops.gemv(Wg, n)), ops.gemv(Wu, n)))
    y = torch.empty(E, dtype=torch.bfloat16, device=cuda)
    K.gemv_fused(dev(Wd), dev(want_m), y, M=E, K=F, residual=dev(x), epilogue=1)
    close(y, ops.add(x, ops.gemv(Wd, want_m)))
    # ... and with the residual's multiplier (AXPY's one fused multiply-add)
    K.gemv_fused(dev(Wd), dev(want_m), y, M=E, K=F, residual=dev(x), residual_scale=0.22, epilogue=1)
    close(y, ops.axpy(0.22, ops.gemv(Wd, want_m), x))
    # the head: norm then projection
    for rows in (4096, 10000, 128256):  # one, two and four rows a wave
        Wh = bf(rows, E, scale=0.02)
        lg = torch.empty(rows, dtype=torch.bfloat16, device=cuda)
        K.gemv_fused(dev(Wh), dev(x), lg, M=rows, K=E, norm_w=dev(g), eps=1e-5, epilogue=0)
        close(lg, ops.gemv(Wh, n))


@pytest.mark.parametrize("E,F,H,G,D", [(4096, 14336, 32, 8, 128), (3072, 8192, 24, 8, 128), (1992, 5000, 3, 1, 64),
                                       (8192, 3000, 8, 8, 128), (264, 16384, 2, 2, 64)])
def test_fused_kernels_at_other_widths(cuda, E, F, H, G, D):
    """The one-row fusions where a row is not the 1B model's: two, four and eight chunks a thread,
    rows whose last chunks a thread has none of (the bounded loads' zeros), an odd count of rows, and
    rows shorter than a block's reach -- each against the oracle's steps composed on the host."""
    import torch

    from iron_amd import kernels as K
    from iron_amd.bf16 import from_torch, round_bf16, to_torch
    from oracle import ops

    rng = np.random.default_rng(E + F)
    L, pos = 16, 5

    def bf(*shape, scale=1.0):
        return round_bf16(rng.standard_normal(shape, dtype=np.float32) * np.float32(scale))

    def dev(a):
        return to_torch(a).to(cuda)

    def close(got, want, atol=2e-2):
        got = from_torch(got).reshape(want.shape)
        assert np.all(np.abs(got - want) <= atol + 1e-2 * np.abs(want)), np.abs(got - want).max()

    x, g = bf(E), round_bf16(rng.uniform(0.9, 1.1, E))
    n = ops.rms_norm(x[None], g, epsilon=1e-5)[0]
    Wq, Wk, Wv = bf(H * D, E, scale=0.02), bf(G * D, E, scale=0.02), bf(G * D, E, scale=0.02)
    table = round_bf16(ops.rope_angles(D, L))
    keys, values = dev(np.zeros((L, G, D), np.float32)), dev(np.zeros((L, G, D), np.float32))
    q_out = torch.empty(H * D, dtype=torch.bfloat16, device=cuda)
    K.decode_qkv(dev(x), dev(g), dev(Wq), dev(Wk), dev(Wv), dev(table), q_out, keys, values, eps=1e-5,
                 hidden=E, heads=H, kv_heads=G, d=D, cache_rows=L,
                 position=torch.tensor([pos], dtype=torch.int32, device=cuda),
                 angle_row=torch.tensor([pos], dtype=torch.int32, device=cuda))
    close(q_out, ops.rope(ops.gemv(Wq, n).reshape(H, D), table[pos : pos + 1]).reshape(-1))
    close(keys[pos], ops.rope(ops.gemv(Wk, n).reshape(G, D), table[pos : pos + 1]))
    close(values[pos], ops.gemv(Wv, n).reshape(G, D))
    Wg, Wu, Wd = bf(F, E, scale=0.02), bf(F, E, scale=0.02), bf(E, F, scale=0.02)
    m = torch.empty(F, dtype=torch.bfloat16, device=cuda)
    K.gemv_fused(dev(Wg), dev(x), m, M=F, K=E, W2=dev(Wu), norm_w=dev(g), eps=1e-5, epilogue=2)
    want_m = ops.mul(ops.silu(ops.gemv(Wg, n)), ops.gemv(Wu, n))
    close(m, want_m)
    y = torch.empty(E, dtype=torch.bfloat16, device=cuda)
    K.gemv_fused(dev(Wd), dev(want_m), y, M=E, K=F, residual=dev(x), epilogue=1)
    close(y, ops.add(x, ops.gemv(Wd, want_m)))
    K.gemv_fused(dev(Wd), dev(want_m), y, M=E, K=F, norm_w=None, epilogue=0)
    close(y, ops.gemv(Wd, want_m))
    row = bf(E)
    K.gemv_fused(dev(Wd), dev(want_m), y, M=E, K=F, residual=dev(row), epilogue=5)
    close(y, ops.mul(ops.silu(ops.gemv(Wd, want_m)), row))


def test_biased_projections_match_hugging_face_on_the_gpu(cuda):
    """q, k, v and o with a bias (RowwiseAdd after each projection) against the reference's second
    golden fixture: prompt, greedy decode under the HIP graph, and a prompt of several chunks."""
    golden, w = Golden(BIASED_GOLDEN), weights(BIASED)
    model = Llama(dataclasses.replace(BIASED, max_seq_len=4 * BIASED.prefill_chunk), w)
    model.load_versions()
    try:
        names = [type(s.op).__name__ for s in model.decode_step.recording.steps]
        assert names.count("RowwiseAdd") == 4 * BIASED.num_hidden_layers
        prompt = np.random.default_rng(1).integers(0, BIASED.vocab_size, 8)
        want = golden.logits(prompt)
        got = model.logits(prompt)
        assert_close(got, want)
        tokens = prompt
        for step in range(6):
            tokens = np.append(tokens, want.argmax())
            want = golden.logits(tokens)
            got = model.logits(tokens)
            assert_close(got, want, f"step {step}")
            assert kl(want, got) < 1e-3
        tokens = np.random.default_rng(3).integers(0, BIASED.vocab_size, BIASED.prefill_chunk + 150)
        assert_close(model.logits(tokens), golden.logits(tokens))
    finally:
        model.release()


def test_a_checkpoint_directory_loads_onto_the_gpu_and_generates_text(cuda, tmp_path, golden):
    """config.json + model.safetensors (bf16 as stored, uploaded without widening) + tokenizer.json."""
    from tests.test_checkpoint import toy_directory

    model = Llama.load(toy_directory(tmp_path))
    try:
        prompt = np.random.default_rng(7).integers(0, SCALED.vocab_size, 8)
        assert_close(model.logits(prompt), golden.logits(prompt))
        ids = model.generate(model.tokenizer("w5 w9"), 5)
        assert model.generate("w5 w9", 5) == model.tokenizer.decode([t for t in ids if t not in model.eos])
    finally:
        model.release()

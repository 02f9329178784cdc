"""The decoder graph on the GPU: compiled versions in one arena, the decode step a HIP graph.

Judged against Hugging Face's float32 logits (the reference's golden fixture) by the
reference's own rule -- within 5 % of the largest logit and the same argmax -- and against
the graph's host reference (the CPU oracle) on the same weights.
"""

import dataclasses

import numpy as np
import pytest

import oracle
from iron_amd.applications.llama import LLAMA_3_2_1B, Llama
from iron_amd.lm.causal import OnHost
from tests.llama_support import SCALED, Golden, assert_close, kl, weights

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


def test_versions_share_one_arena_and_the_decode_step_is_a_hip_graph(toy):
    decode, prompt = toy.decode_step, toy.prompt_chunk
    assert decode.arena is prompt.arena and decode.arena.buffer is not None
    assert decode.captured and not prompt.captured
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

"""The decoder graph's host reference against Hugging Face's float32 forward pass.

The reference's own golden logits (tests/golden/llama_small_hf_logits.npz) judge the graph
wiring -- layouts, reshapes, head grouping, RoPE convention and scaling, the caches a prompt
leaves for decode, chunked prefill -- with the oracle's operator references underneath and no
GPU (iron/tests/common/test_llama_reference.py, iron/tests/support/llama_reference.py:86-251).
"""

import dataclasses

import numpy as np
import pytest

import oracle
from iron_amd.applications.llama import Llama
from iron_amd.lm.causal import OnHost
from tests.llama_support import BIASED, BIASED_GOLDEN, SCALED, Golden, assert_close, kl, weights

oracle.install()


class HostLlama(OnHost, Llama):
    pass


@pytest.fixture(scope="module")
def golden():
    return Golden()


@pytest.fixture(scope="module")
def w():
    return weights()


def host(config, w):
    model = HostLlama(config, w)
    model.load_versions()
    return model


def greedy_case(golden, seed=7):
    prompt = np.random.default_rng(seed).integers(0, SCALED.vocab_size, 8)
    tokens, expected = prompt, []
    first = logits = golden.logits(tokens)
    for _ in range(6):
        tokens = np.append(tokens, logits.argmax())
        logits = golden.logits(tokens)
        expected.append(logits)
    return prompt, first, expected


def test_golden_fixture_is_the_reference_s():
    g = Golden()
    prompt = np.random.default_rng(7).integers(0, 1024, 8)
    first = g.logits(prompt)
    # The row the survey reproduced bit for bit from HF: argmax 374, max |logit| 3.1666.
    assert first.shape == (1024,) and int(first.argmax()) == 374 and abs(np.abs(first).max() - 3.1666) < 1e-3


def test_the_prompt_matches_the_forward_and_leaves_decode_its_caches(golden, w):
    prompt, first, expected = greedy_case(golden)
    model = host(SCALED, w)
    got = model.logits(prompt)
    assert_close(got, first)
    tokens = prompt
    for step, want in enumerate(expected):
        tokens = np.append(tokens, got.argmax())
        got = model.logits(tokens)
        assert_close(got, want, f"step {step}")


def test_decode_from_an_empty_cache_matches_the_forward_token_by_token(golden, w):
    prompt, first, expected = greedy_case(golden)
    model = host(SCALED, w)
    for n in range(1, len(prompt) + 1):
        last = model.logits(prompt[:n])
    assert_close(last, first)
    assert kl(first, last) < 1e-3


def test_a_prompt_longer_than_a_chunk_runs_in_chunks(golden, w):
    C = SCALED.prefill_chunk
    config = dataclasses.replace(SCALED, max_seq_len=4 * C)
    model = host(config, w)
    tokens = np.random.default_rng(3).integers(0, config.vocab_size, C + 150)
    first = golden.logits(tokens)
    assert_close(model.logits(tokens), first)
    tokens = np.append(tokens, first.argmax())
    assert_close(model.logits(tokens), golden.logits(tokens))
    turn = np.random.default_rng(4).integers(0, config.vocab_size, 30)
    tokens = np.append(tokens, turn)
    assert_close(model.logits(tokens), golden.logits(tokens))


@pytest.mark.parametrize("outside", [-1, SCALED.vocab_size])
def test_a_token_outside_the_vocabulary_is_refused_before_any_dispatch(w, outside):
    model = host(dataclasses.replace(SCALED, prefill_chunk=64), w)
    tokens = np.random.default_rng(6).integers(0, SCALED.vocab_size, 100)
    model.logits(tokens)
    broken = tokens.copy()
    broken[3] = (broken[3] + 1) % SCALED.vocab_size
    broken[70] = outside
    with pytest.raises(IndexError, match=rf"\[{outside}\] are outside"):
        model.logits(broken)
    np.testing.assert_array_equal(model.session.cached, tokens)


def test_a_model_runs_only_the_versions_it_loaded(w):
    model = Llama(SCALED, w)
    with pytest.raises(RuntimeError, match=r"load_versions\(\) first"):
        model.logits([1, 2, 3])
    with pytest.raises(RuntimeError, match=r"load_versions\(\) first"):
        model(start=0, rows=1, rope_start=0, token=0, position=0)


# ---- projections with a bias (RowwiseAdd), against the reference's second golden fixture
def test_biased_projections_match_the_forward_prompt_then_decode():
    golden, w = Golden(BIASED_GOLDEN), weights(BIASED)
    prompt, first, expected = greedy_case(golden, seed=1)
    model = host(BIASED, w)
    got = model.logits(prompt)
    assert_close(got, first)
    assert kl(first, got) < 1e-3
    tokens = prompt
    for step, want in enumerate(expected):
        tokens = np.append(tokens, got.argmax())
        got = model.logits(tokens)
        assert_close(got, want, f"step {step}")


def test_biased_projections_match_the_forward_token_by_token_and_in_chunks():
    golden, w = Golden(BIASED_GOLDEN), weights(BIASED)
    prompt, first, _ = greedy_case(golden, seed=1)
    model = host(BIASED, w)
    for n in range(1, len(prompt) + 1):
        last = model.logits(prompt[:n])
    assert_close(last, first)
    C = BIASED.prefill_chunk
    model = host(dataclasses.replace(BIASED, max_seq_len=4 * C), w)
    tokens = np.random.default_rng(3).integers(0, BIASED.vocab_size, C + 150)
    assert_close(model.logits(tokens), golden.logits(tokens))


def test_a_bias_changes_the_logits():
    """The biased toy's weights with the biases dropped no longer match its golden: the bias is used."""
    golden, w = Golden(BIASED_GOLDEN), weights(BIASED)
    prompt, first, _ = greedy_case(golden, seed=1)
    zeroed = {n: (np.zeros_like(a) if n.endswith("bias") else a) for n, a in w.items()}
    got = host(BIASED, zeroed).logits(prompt)
    assert np.abs(np.asarray(got, np.float32).reshape(-1) - first).max() > 0.05 * np.abs(first).max()


def test_a_sampler_s_rows_draw_on_the_graph_what_the_sampler_draws_on_the_host(w):
    """``generate`` with a sampler writes one draw row per position ahead of time and the graph's
    Sample draws from them; the same sampler called on each step's logits draws the same tokens
    (iron/lm/testing.py:169-179)."""
    from iron_amd.lm.generation import Sampler, generate_on_host

    prompt = np.random.default_rng(12).integers(0, SCALED.vocab_size, 8)
    model = host(SCALED, w)
    drawn = model.generate(prompt, 5, Sampler(1.5, 50, seed=2))
    assert drawn == generate_on_host(model, prompt, 5, Sampler(1.5, 50, seed=2))
    greedy = model.generate(prompt, 5)
    assert greedy == generate_on_host(model, prompt, 5, Sampler(0.0))
    assert drawn != greedy   # at this temperature the toy's flat logits do not keep to the top token

"""Granite's graph against Hugging Face's Granite in float32 over the same random weights at a toy
shape: the reference's own fixture (tests/applications/granite/reference/goldens/toy.npz, committed
as tests/golden/granite_toy_hf_logits.npz) with Granite's four scalars, none at its default, and an
untied head (tests/applications/granite/reference/test.py:15-44).  On the host through the oracle's
operator references, and compiled on the GPU.
"""

from pathlib import Path

import numpy as np
import pytest

import oracle
from iron_amd.applications.granite import Granite, GraniteConfig, shapes
from iron_amd.lm.causal import OnHost
from oracle import ops
from tests.llama_support import Golden, assert_close

oracle.install()

TOY = GraniteConfig(
    vocab_size=1024, hidden_size=512, num_hidden_layers=2, num_attention_heads=8, num_key_value_heads=2,
    intermediate_size=1024, rope_theta=10000.0, max_seq_len=256, prefill_chunk=256, tie_word_embeddings=False,
    attention_multiplier=0.0625, residual_multiplier=0.22, embedding_multiplier=12.0, logits_scaling=8.0,
)
GOLDEN = Path(__file__).parent / "golden" / "granite_toy_hf_logits.npz"


class HostGranite(OnHost, Granite):
    pass


@pytest.fixture(scope="module")
def golden():
    return Golden(GOLDEN)


@pytest.fixture(scope="module")
def w():
    return ops.filled(shapes(TOY), seed=0)


def case(golden):
    """The prompt (seed 0, as the reference's test draws it), its logits and six greedy steps'."""
    prompt = np.random.default_rng(0).integers(0, TOY.vocab_size, 8)
    tokens, expected = prompt, []
    first = logits = golden.logits(tokens)
    for _ in range(6):
        tokens = np.append(tokens, logits.argmax())
        logits = golden.logits(tokens)
        expected.append(logits)
    return prompt, first, expected


def greedy_against(model, golden):
    prompt, first, expected = case(golden)
    got = model.logits(prompt)
    assert_close(got, first, "the prompt")
    tokens = prompt
    for step, want in enumerate(expected):
        tokens = np.append(tokens, got.argmax())
        got = model.logits(tokens)
        assert_close(got, want, f"step {step}")


def test_the_scalars_are_read_from_a_config_json():
    data = TOY.to_json()
    assert data["attention_multiplier"] == 0.0625 and data["logits_scaling"] == 8.0
    again = GraniteConfig.from_json(data)
    assert again.residual_multiplier == 0.22 and again.embedding_multiplier == 12.0 and not again.tie_word_embeddings
    with pytest.raises(ValueError, match="attention_multiplier"):
        GraniteConfig.from_json({k: v for k, v in data.items() if k != "attention_multiplier"})


def test_the_prompt_and_greedy_decode_match_hugging_face_on_the_host(golden, w):
    model = HostGranite(TOY, w)
    model.load_versions()
    greedy_against(model, golden)


def test_decode_from_an_empty_cache_matches_token_by_token_on_the_host(golden, w):
    model = HostGranite(TOY, w)
    model.load_versions()
    prompt, first, _ = case(golden)
    for n in range(1, len(prompt) + 1):
        last = model.logits(prompt[:n])
    assert_close(last, first)


def test_every_scalar_matters(golden, w):
    """Each of the four scalars at its default moves the logits away from the golden's."""
    import dataclasses

    prompt, first, _ = case(golden)
    for field in ("attention_multiplier", "residual_multiplier", "embedding_multiplier", "logits_scaling"):
        model = HostGranite(dataclasses.replace(TOY, **{field: 1.0}), w)
        model.load_versions()
        with pytest.raises(AssertionError):
            assert_close(model.logits(prompt), first)


@pytest.mark.gpu
def test_the_compiled_graph_matches_hugging_face_on_the_gpu(cuda, golden, w):
    model = Granite(TOY, w)
    model.load_versions()
    try:
        assert model.decode_step.captured
        greedy_against(model, golden)
        # The device-carried run draws what stepwise decode draws.
        prompt, _, _ = case(golden)
        assert model.generate(prompt, 12) == list(model.session.draw(prompt, 12, each=True))
        names = [type(s.op).__name__ for s in model.decode_step.recording.steps]
        assert names.count("AXPY") == 2 * TOY.num_hidden_layers and "RowwiseMul" in names
        # The scaled residuals ride the fused GEMVs' epilogue: five launches a layer, as Llama's; the
        # embedding's gather, its multiplier, the head (norm + GEMV) and the draw (the RoPE row is read from
        # its table by the projections' launch).
        assert model.decode_step.launches_per_call == 2 + 5 * TOY.num_hidden_layers + 2
    finally:
        model.release()


@pytest.mark.gpu
def test_fused_and_step_by_step_launches_agree(cuda, golden, w):
    fused, plain = Granite(TOY, w), Granite(TOY, w)
    fused.load_versions(fuse=True)
    plain.load_versions(fuse=False)
    try:
        assert plain.decode_step.launches_per_call == len(plain.decode_step.recording.steps)
        prompt, _, _ = case(golden)
        tokens = prompt
        for step in range(6):
            a, b = fused.logits(tokens), plain.logits(tokens)
            assert np.abs(a - b).max() <= 0.02 * np.abs(b).max(), step
            tokens = np.append(tokens, golden.logits(tokens).argmax())
        assert fused.generate(prompt, 24) == plain.generate(prompt, 24)
    finally:
        fused.release()
        plain.release()

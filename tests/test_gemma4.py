"""Gemma 4's text decoder against Hugging Face's Gemma 4 in float32 over the same random weights at
a toy shape: the reference's own fixture (tests/applications/gemma4/reference/goldens/toy.npz,
committed as tests/golden/gemma4_toy_hf_logits.npz).  The toy has Gemma 4 E2B's proportions
(tests/applications/gemma4/reference/test.py:22-47): one KV head, sliding and global layers
alternating, global layers of their own head size and proportional RoPE, the last two layers
sharing caches (a sliding and a global one), double-wide MLPs, per-layer inputs, capped logits, and
a context past three rings so the sliding layers keep a ring.  On the host through the oracle's
operator references, and compiled on the GPU.
"""

import dataclasses
from pathlib import Path

import numpy as np
import pytest

import oracle
from iron_amd.applications.gemma4 import Gemma4, Gemma4Config, shapes
from iron_amd.bf16 import round_bf16
from iron_amd.lm.causal import OnHost
from oracle import ops
from tests.llama_support import Golden, assert_close

oracle.install()

TOY = Gemma4Config(
    vocab_size=1024, hidden_size=512, num_hidden_layers=6, num_attention_heads=4, num_key_value_heads=1,
    head_dim=128, intermediate_size=512, rope_theta=10000.0, max_seq_len=512, prefill_chunk=64,
    sliding_window=8, layer_types=("sliding_attention", "full_attention") * 3, global_head_dim=256,
    num_kv_shared_layers=2, use_double_wide_mlp=True, ple_dim=128, final_logit_softcapping=5.0,
)
GOLDEN = Path(__file__).parent / "golden" / "gemma4_toy_hf_logits.npz"


class HostGemma4(OnHost, Gemma4):
    pass


@pytest.fixture(scope="module")
def golden():
    return Golden(GOLDEN)


def weights(config=TOY):
    """The drawn tensors, q's and k's norms each scaled by ``head_dim ** -0.25``: attention is
    unscaled, so a trained model's norms carry the ``head_dim ** -0.5`` that unit norms leave out
    (tests/applications/gemma4/reference/test.py:110-122)."""
    w = ops.filled(shapes(config), seed=0)
    for name, weight in w.items():
        if name.endswith(("q_norm.weight", "k_norm.weight")):
            w[name] = round_bf16(weight.astype(np.float32) * np.float32(weight.size**-0.25))
    return w


@pytest.fixture(scope="module")
def w():
    return weights()


def host(config, w):
    model = HostGemma4(config, w)
    model.load_versions()
    return model


def case(golden, seed=7):
    """The prompt (as the reference's test draws it), its logits and six greedy steps'."""
    prompt = np.random.default_rng(seed).integers(0, TOY.vocab_size, 8)
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


def chunks_against(model, golden, config):
    """A prompt of several chunks, a decode step, then a turn of 30 tokens, which reruns only the
    chunk holding its first token onwards (iron/tests/support/llama_reference.py:208-226)."""
    C = TOY.prefill_chunk
    tokens = np.random.default_rng(3).integers(0, config.vocab_size, C + 150)
    first = golden.logits(tokens)
    assert_close(model.logits(tokens), first, "the chunks")
    tokens = np.append(tokens, first.argmax())
    assert_close(model.logits(tokens), golden.logits(tokens), "the step after")
    turn = np.random.default_rng(4).integers(0, config.vocab_size, 30)
    tokens = np.append(tokens, turn)
    assert_close(model.logits(tokens), golden.logits(tokens), "the turn")


def test_the_toy_keeps_rings_and_shares_caches(w):
    model = HostGemma4(TOY, w)
    c = TOY
    assert [c.owner(i) for i in range(6)] == [0, 1, 2, 3, 2, 3]
    rings = [layer.cache.ring for layer in model.layers]
    assert rings == [128, None, 128, None, 128, None]
    assert model.layers[4].cache is model.layers[2].cache and model.layers[5].cache is model.layers[3].cache
    assert model.layers[4].self_attn.k_proj is None and model.layers[3].self_attn.k_proj is not None
    assert len(model.recurrent) == 2
    assert model.layers[4].mlp.gate_proj.out_features == 2 * c.intermediate_size
    assert model.layers[1].self_attn.head_dim == 256 and model.layers[0].self_attn.head_dim == 128


def test_the_config_is_read_from_a_config_json():
    data = TOY.to_json()
    text = data["text_config"]
    assert text["rope_parameters"]["full_attention"]["rope_theta"] == 1000000.0
    assert text["hidden_size_per_layer_input"] == 128 and text["hidden_activation"] == "gelu_pytorch_tanh"
    again = Gemma4Config.from_json(data)
    assert dataclasses.replace(again, prefill_chunk=TOY.prefill_chunk) == TOY
    for refused in ({"attention_k_eq_v": True}, {"enable_moe_block": True}, {"use_bidirectional_attention": "all"},
                    {"use_bidirectional_attention": True}, {"attn_logit_softcapping": 50.0},
                    {"vocab_size_per_layer_input": 512},
                    {"rope_parameters": {"full_attention": {"rope_type": "default"}}}):
        changed = {**data, "text_config": {**text, **refused}}
        with pytest.raises(ValueError, match="not built here"):
            Gemma4Config.from_json(changed)
    # Bidirectional attention for images alone is text's causal.
    Gemma4Config.from_json({**data, "text_config": {**text, "use_bidirectional_attention": "vision"}})


def test_the_prompt_and_greedy_decode_match_hugging_face_on_the_host(golden, w):
    greedy_against(host(TOY, w), golden)


def test_decode_from_an_empty_cache_matches_token_by_token_on_the_host(golden, w):
    model = host(TOY, w)
    prompt, first, _ = case(golden)
    for n in range(1, len(prompt) + 1):
        last = model.logits(prompt[:n])
    assert_close(last, first)


def test_a_prompt_longer_than_a_chunk_runs_in_chunks_on_the_host(golden, w):
    # Four chunks of context: no ring (tests/applications: the reference's own chunked case).
    config = dataclasses.replace(TOY, max_seq_len=4 * TOY.prefill_chunk)
    model = host(config, w)
    assert all(layer.cache.ring is None for layer in model.layers)
    chunks_against(model, golden, config)


def test_the_rings_give_the_same_logits_on_the_host(golden, w):
    # The toy's own context: the sliding layers' rings (128 rows) wrap within the 245 positions.
    model = host(TOY, w)
    chunks_against(model, golden, TOY)


@pytest.mark.gpu
def test_the_compiled_graph_matches_hugging_face_on_the_gpu(cuda, golden, w):
    model = Gemma4(TOY, w)
    model.load_versions()
    try:
        assert model.decode_step.captured
        greedy_against(model, golden)
        chunks_against(model, golden, TOY)
        prompt, _, _ = case(golden)
        assert model.generate(prompt, 12) == list(model.session.draw(prompt, 12, each=True))
        # Replays whose ring rows the device derives from the carried position, across the wrap
        # (positions 100 .. 159 over rings of 128 rows), against steps whose words the host wrote.
        long = np.random.default_rng(12).integers(0, TOY.vocab_size, 100)
        assert model.generate(long, 60) == list(model.session.draw(long, 60, each=True))
    finally:
        model.release()


@pytest.mark.gpu
@pytest.mark.parametrize("global_head_dim", [256, 512])   # 512: Gemma 4 E2B's own global heads
def test_the_gpu_matches_the_host_step_by_step_past_a_ring(cuda, global_head_dim):
    config = dataclasses.replace(TOY, global_head_dim=global_head_dim)
    w = weights(config)
    gpu, cpu = Gemma4(config, w), host(config, w)
    gpu.load_versions()
    try:
        tokens = np.random.default_rng(11).integers(0, TOY.vocab_size, 300)
        for n in (150, 151, 152, 300):
            got, want = gpu.logits(tokens[:n]), cpu.logits(tokens[:n])
            assert np.abs(got - want).max() <= 0.03 * np.abs(want).max(), n
        # Logits bitwise the same run after run, over rings that wrap and alternating prompts.
        from iron_amd.lm.generation import determinism

        assert determinism(gpu, [tokens[:150], tokens[40:200]], 3, rounds=2) == 0
    finally:
        gpu.release()


@pytest.mark.gpu
def test_the_fused_decode_step_matches_the_step_by_step_one(cuda, w):
    """The one-row fusions of Gemma 4's layers -- the input norm riding the q, k, v projections, the
    per-head norms, RoPE and cache rows (ring and mirror) as one launch, the per-layer input's gate in
    its projection's epilogue -- against every recorded step launched on its own: the same logits
    within bf16 rounding across a ring's wrap, in well under three quarters of the launches."""
    fused, plain = Gemma4(TOY, w), Gemma4(TOY, w)
    fused.load_versions(fuse=True)
    plain.load_versions(fuse=False)
    try:
        steps = len(plain.decode_step.recording.steps)
        assert plain.decode_step.launches_per_call == steps
        assert fused.decode_step.launches_per_call <= 0.6 * steps
        tokens = np.random.default_rng(14).integers(0, TOY.vocab_size, 140)
        for n in (30, 31, 32, 139, 140):     # prompt chunks, then single decode steps; the rings hold 128 rows
            a, b = fused.logits(tokens[:n]), plain.logits(tokens[:n])
            assert np.abs(a - b).max() <= 0.02 * np.abs(b).max(), n
        assert fused.generate(tokens[:100], 40) == list(fused.session.draw(tokens[:100], 40, each=True))
    finally:
        fused.release()
        plain.release()


@pytest.mark.gpu
def test_check_mode_judges_every_step_of_gemma_against_its_reference(cuda, w):
    """Every recorded step launched on its own and judged against its operator's reference by the
    operator's own tolerance: the per-head norms, GELU, the capped logits and the constant rows too."""
    model = Gemma4(TOY, w)
    model.load_versions(check=True)
    try:
        prompt = np.random.default_rng(9).integers(0, TOY.vocab_size, 70)   # two chunks
        model.logits(prompt)
        model.logits(np.append(prompt, 5))
    finally:
        model.release()

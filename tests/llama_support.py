"""The toy Llama of the reference's device-free model tests and its recorded HF logits.

``SCALED``: hidden 512, 2 layers, 16 q / 4 kv heads, head_dim 64, intermediate 2048,
vocab 1024, theta 5e5, eps 1e-5, Llama-3 RoPE scaling factor 8 from a 64-position original
context (iron/tests/support/llama_model.py:56-68, iron/tests/common/test_llama_reference.py:52-60).
Weights are the reference's random draw at seed 0 (iron/common/graph/fill.py:13-33), restated
in the oracle.  ``tests/golden/llama_small_hf_logits.npz`` is the reference's own fixture
(iron/tests/common/goldens/small.npz): float32 logits of Hugging Face's LlamaForCausalLM on
those weights, keyed by sha256(int64 tokens)[:16] (iron/lm/golden.py:88-92).
"""

import dataclasses
import hashlib
from pathlib import Path

import numpy as np

from iron_amd.applications.llama import Llama3RopeScaling, LlamaConfig, shapes
from oracle import ops

GOLDEN = Path(__file__).parent / "golden" / "llama_small_hf_logits.npz"

SCALED = LlamaConfig(
    vocab_size=1024, hidden_size=512, num_hidden_layers=2, num_attention_heads=16, num_key_value_heads=4,
    head_dim=64, intermediate_size=2048, rope_theta=500000.0, max_seq_len=256, prefill_chunk=256, eps=1e-5,
    rope_scaling=Llama3RopeScaling(factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                   original_max_position_embeddings=64),
)


# The reference's second toy: the same shape with its RoPE table unscaled and a bias on each of
# q, k, v and o (tests/applications/llama/reference/test.py:23-43; SMALL,
# iron/tests/support/llama_model.py:56-68).  Its golden, tests/golden/llama_biased_hf_logits.npz,
# is the reference's tests/applications/llama/reference/goldens/biased.npz; prompts are drawn at seed 1.
BIASED = dataclasses.replace(SCALED, rope_scaling=None, attention_bias=True)
BIASED_GOLDEN = Path(__file__).parent / "golden" / "llama_biased_hf_logits.npz"


def biased_names(config=BIASED):
    """The checkpoint's names in the order the reference's test draws them: Llama's, then each
    layer's four biases."""
    c = config
    Q, KV = c.num_attention_heads * c.head_dim, c.num_key_value_heads * c.head_dim
    out = dict(shapes(c))
    for i in range(c.num_hidden_layers):
        attention = f"model.layers.{i}.self_attn"
        out |= {f"{attention}.q_proj.bias": (Q,), f"{attention}.k_proj.bias": (KV,),
                f"{attention}.v_proj.bias": (KV,), f"{attention}.o_proj.bias": (c.hidden_size,)}
    return out


def weights(config=SCALED, seed=0):
    named = biased_names(config) if config.attention_bias else shapes(config)
    return ops.filled(named, seed=seed)


class Golden:
    def __init__(self, path=GOLDEN):
        z = np.load(path)
        self.rows = {k: z[k] for k in z.files if k != "fingerprint"}

    def logits(self, tokens) -> np.ndarray:
        key = hashlib.sha256(np.asarray(tokens, dtype=np.int64).reshape(-1).tobytes()).hexdigest()[:16]
        if key not in self.rows:
            raise LookupError(f"the golden holds no logits for these {len(tokens)} tokens")
        return self.rows[key]


def assert_close(got, want, what="the logits", share=0.05):
    """``got`` within ``share`` of the reference's largest logit, and the same argmax where the
    reference's top two differ by more than that (iron/lm/testing.py:182-206)."""
    got = np.asarray(got, np.float32).reshape(want.shape)
    scale = np.abs(want).max()
    bound, err = share * scale, np.abs(got - want).max()
    assert err <= bound, f"{what}: max |diff| {err:.4f} against |logits| {scale:.3f}"
    second, first = np.sort(want, axis=None)[-2:]
    if first - second > bound:
        assert got.argmax() == want.argmax(), f"{what}: argmax {got.argmax()} != {want.argmax()}"


def kl(reference_logits, logits) -> float:
    """KL(reference || model) of the two next-token distributions."""
    p = reference_logits.astype(np.float64)
    q = np.asarray(logits, np.float64).reshape(p.shape)
    p = p - p.max()
    q = q - q.max()
    lp, lq = p - np.log(np.exp(p).sum()), q - np.log(np.exp(q).sum())
    return float((np.exp(lp) * (lp - lq)).sum())

"""Llama 3 on the shared decoder: its RoPE scaling and Llama 3.2 1B's shape
(iron/applications/llama/model.py:22-103)."""

from __future__ import annotations

import dataclasses

import numpy as np

from ..common.declare import Precision
from ..lm import CausalLM, DecoderConfig


@dataclasses.dataclass(frozen=True)
class Llama3RopeScaling:
    """The ``"rope_type": "llama3"`` entry of a config: long wavelengths are slowed by ``factor``,
    short ones kept, and the band between the two cut-offs (``original_max_position_embeddings``
    over ``low_freq_factor`` / ``high_freq_factor``) blends from one to the other."""

    factor: float
    low_freq_factor: float
    high_freq_factor: float
    original_max_position_embeddings: int
    rope_type: str = "llama3"

    def __call__(self, inv_freq: np.ndarray) -> np.ndarray:
        """The scaled inverse frequencies, elementwise, in ``inv_freq``'s own precision."""
        context = self.original_max_position_embeddings
        wavelength = 2 * np.pi / inv_freq
        # 0 at the low cut-off, 1 at the high one: the share of the unscaled frequency in the blend
        share = (context / wavelength - self.low_freq_factor) / (self.high_freq_factor - self.low_freq_factor)
        blended = (1 - share) * inv_freq / self.factor + share * inv_freq
        slowed = np.where(wavelength > context / self.low_freq_factor, inv_freq / self.factor, blended)
        return np.where(wavelength < context / self.high_freq_factor, inv_freq, slowed)

    @classmethod
    def from_dict(cls, data: dict) -> "Llama3RopeScaling":
        """From a config's ``rope_scaling`` mapping.

        Raises:
            ValueError: another ``rope_type`` than ``llama3``.
        """
        kind = data.get("rope_type")
        if kind != "llama3":
            raise ValueError(f"rope_scaling {data}: no RoPE table here builds it")
        return cls(**data)


@dataclasses.dataclass(frozen=True)
class LlamaConfig(DecoderConfig):
    """A decoder's config whose ``rope_scaling`` is Llama 3's."""

    rope_scaling: Llama3RopeScaling | None = None
    precision: Precision = Precision.MEDIUM

    @classmethod
    def convert(cls, name: str, value):
        return Llama3RopeScaling.from_dict(value) if name == "rope_scaling" else super().convert(name, value)

    @classmethod
    def from_json(cls, data: dict, source="config.json") -> "LlamaConfig":
        """``DecoderConfig.from_json``; models as wide as Llama 3.2 3B or wider ask for
        ``Precision.HIGH`` as the reference does for its device (here every precision runs the same
        float32-accumulating kernels, so the field is carried, not acted on)."""
        parsed = super().from_json(data, source)
        wide = parsed.hidden_size >= 3072
        return dataclasses.replace(parsed, precision=Precision.HIGH) if wide else parsed


LLAMA_3_2_1B = LlamaConfig(   # the shape of meta-llama/Llama-3.2-1B
    vocab_size=128256, hidden_size=2048, num_hidden_layers=16, num_attention_heads=32,
    num_key_value_heads=8, head_dim=64, intermediate_size=8192, rope_theta=500000.0,
    max_seq_len=131072, eps=1e-5,
    rope_scaling=Llama3RopeScaling(factor=32.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                   original_max_position_embeddings=8192),
)

# A layer's tensors in checkpoint order: name under ``model.layers.<i>.`` and (rows, columns) as
# letters -- E hidden, Q all query heads, K all KV heads, F the feed-forward's width; one letter is a vector.
_LAYER_TENSORS = (
    ("input_layernorm", "E"), ("self_attn.q_proj", "QE"), ("self_attn.k_proj", "KE"), ("self_attn.v_proj", "KE"),
    ("self_attn.o_proj", "EQ"), ("post_attention_layernorm", "E"), ("mlp.gate_proj", "FE"), ("mlp.up_proj", "FE"),
    ("mlp.down_proj", "EF"),
)


def shapes(config: DecoderConfig) -> dict[str, tuple[int, ...]]:
    """Name -> shape of every tensor in a Hugging Face Llama checkpoint of this config, in the
    checkpoint's order (the order a seeded weight draw follows: iron/tests/support/llama_model.py:76-98)."""
    size = {"E": config.hidden_size, "F": config.intermediate_size,
            "Q": config.num_attention_heads * config.head_dim, "K": config.num_key_value_heads * config.head_dim}
    named = {"model.embed_tokens.weight": (config.vocab_size, size["E"]), "model.norm.weight": (size["E"],)}
    for index in range(config.num_hidden_layers):
        for tensor, letters in _LAYER_TENSORS:
            named[f"model.layers.{index}.{tensor}.weight"] = tuple(size[letter] for letter in letters)
    return named


class Llama(CausalLM):
    """Llama 3: the shared decoder as it stands, configured by a ``LlamaConfig``; ``weights`` is a
    checkpoint's tensors by name."""

    config_class = LlamaConfig

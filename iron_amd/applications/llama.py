"""Llama 3 on the shared decoder: its RoPE scaling and Llama 3.2 1B's shape
(iron/applications/llama/model.py:22-103)."""

from __future__ import annotations

import dataclasses

import numpy as np

from ..common.declare import Precision
from ..lm import CausalLM, DecoderConfig


@dataclasses.dataclass(frozen=True)
class Llama3RopeScaling:
    """Llama 3's RoPE frequency scaling (``"rope_type": "llama3"``)."""

    factor: float
    low_freq_factor: float
    high_freq_factor: float
    original_max_position_embeddings: int
    rope_type: str = "llama3"

    def __call__(self, inv_freq: np.ndarray) -> np.ndarray:
        original = self.original_max_position_embeddings
        wavelen = 2 * np.pi / inv_freq
        smooth = (original / wavelen - self.low_freq_factor) / (self.high_freq_factor - self.low_freq_factor)
        between = (1 - smooth) * inv_freq / self.factor + smooth * inv_freq
        return np.where(
            wavelen < original / self.high_freq_factor,
            inv_freq,
            np.where(wavelen > original / self.low_freq_factor, inv_freq / self.factor, between),
        )

    @classmethod
    def from_dict(cls, data: dict) -> "Llama3RopeScaling":
        if data.get("rope_type") != "llama3":
            raise ValueError(f"rope_scaling {data}: no RoPE table here builds it")
        return cls(**data)


@dataclasses.dataclass(frozen=True)
class LlamaConfig(DecoderConfig):
    """``DecoderConfig`` with Llama 3's own ``rope_scaling``."""

    rope_scaling: Llama3RopeScaling | None = None
    precision: Precision = Precision.MEDIUM

    @classmethod
    def convert(cls, name: str, value):
        if name == "rope_scaling":
            return Llama3RopeScaling.from_dict(value)
        return super().convert(name, value)

    @classmethod
    def from_json(cls, data: dict, source="config.json") -> "LlamaConfig":
        """As ``DecoderConfig.from_json``, at ``Precision.HIGH`` from 3B's width up (the reference's
        choice for its device; every precision runs the same f32-accumulating kernels here)."""
        config = super().from_json(data, source)
        if config.hidden_size < 3072:
            return config
        return dataclasses.replace(config, precision=Precision.HIGH)


#: Llama 3.2 1B's shape.
LLAMA_3_2_1B = LlamaConfig(
    vocab_size=128256, hidden_size=2048, num_hidden_layers=16, num_attention_heads=32,
    num_key_value_heads=8, head_dim=64, intermediate_size=8192, rope_theta=500000.0,
    max_seq_len=131072, eps=1e-5,
    rope_scaling=Llama3RopeScaling(factor=32.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                   original_max_position_embeddings=8192),
)


def shapes(config: DecoderConfig) -> dict[str, tuple[int, ...]]:
    """Each tensor of a Hugging Face Llama checkpoint of ``config``'s shape, by name, in the
    checkpoint's order (iron/tests/support/llama_model.py:76-98)."""
    c = config
    E, F, V = c.hidden_size, c.intermediate_size, c.vocab_size
    Q, KV = c.num_attention_heads * c.head_dim, c.num_key_value_heads * c.head_dim
    out = {"model.embed_tokens.weight": (V, E), "model.norm.weight": (E,)}
    for i in range(c.num_hidden_layers):
        layer = f"model.layers.{i}"
        out |= {
            f"{layer}.input_layernorm.weight": (E,),
            f"{layer}.self_attn.q_proj.weight": (Q, E),
            f"{layer}.self_attn.k_proj.weight": (KV, E),
            f"{layer}.self_attn.v_proj.weight": (KV, E),
            f"{layer}.self_attn.o_proj.weight": (E, Q),
            f"{layer}.post_attention_layernorm.weight": (E,),
            f"{layer}.mlp.gate_proj.weight": (F, E),
            f"{layer}.mlp.up_proj.weight": (F, E),
            f"{layer}.mlp.down_proj.weight": (E, F),
        }
    return out


class Llama(CausalLM):
    """Llama 3 on ``config``'s shape and a checkpoint's ``weights`` (a dict by tensor name)."""

    config_class = LlamaConfig

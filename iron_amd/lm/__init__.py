"""A decoder-only language model wired from the hot-path operators (iron/lm/__init__.py)."""

from .blocks import (
    Attention,
    DecoderLayer,
    Embedding,
    GatedMLP,
    KVCache,
    Linear,
    PleLayer,
    RMSNorm,
    Rope,
    SandwichLayer,
    activation,
    residual_add,
)
from .causal import Call, CausalLM, Decoder, Stats
from .checkpoint import Checkpoint, weights_file, write_safetensors
from .config import DecoderConfig, rope_angles
from .generation import Sampler
from .session import Session

__all__ = [
    "Attention", "Call", "CausalLM", "Checkpoint", "Decoder", "DecoderConfig", "DecoderLayer", "Embedding", "GatedMLP",
    "KVCache", "Linear", "PleLayer", "RMSNorm", "Rope", "Sampler", "SandwichLayer", "Session", "Stats", "activation",
    "residual_add", "rope_angles", "weights_file", "write_safetensors",
]

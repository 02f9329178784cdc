"""A decoder-only language model wired from the hot-path operators."""

from .causal import Call, CausalLM, Decoder, Stats
from .checkpoint import Checkpoint, weights_file, write_safetensors
from .config import DecoderConfig, rope_angles
from .generation import Sampler
from .session import Session

__all__ = ["Call", "CausalLM", "Checkpoint", "Decoder", "DecoderConfig", "Sampler", "Session", "Stats", "rope_angles",
           "weights_file", "write_safetensors"]

"""A decoder-only language model wired from the hot-path operators."""

from .causal import Call, CausalLM, Decoder, Stats
from .config import DecoderConfig, rope_angles
from .session import Session

__all__ = ["Call", "CausalLM", "Decoder", "DecoderConfig", "Session", "Stats", "rope_angles"]

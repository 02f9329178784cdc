"""Granite on the shared decoder (iron/applications/granite/model.py:22-85).

Granite is Llama's layer with four scalars from its config: attention scaled by
``attention_multiplier``, each block's output by ``residual_multiplier`` before its residual
(``GraniteLayer``), the embedding rows by ``embedding_multiplier`` and the logits divided by
``logits_scaling``.  Its head is untied (``lm_head``).
"""

from __future__ import annotations

import dataclasses
import math

import numpy as np

from ..bf16 import from_torch, round_bf16
from ..common import graph as iron
from ..common.declare import Precision
from ..lm import CausalLM, DecoderConfig
from ..lm.blocks import DecoderLayer


@dataclasses.dataclass(frozen=True)
class GraniteConfig(DecoderConfig):
    """``DecoderConfig`` and Granite's own four scalars."""

    attention_multiplier: float = dataclasses.field(kw_only=True)
    residual_multiplier: float = dataclasses.field(default=1.0, kw_only=True)
    embedding_multiplier: float = dataclasses.field(default=1.0, kw_only=True)
    logits_scaling: float = dataclasses.field(default=1.0, kw_only=True)
    precision: Precision = dataclasses.field(default=Precision.HIGH, kw_only=True)


class GraniteLayer(DecoderLayer):
    """Llama's layer, its attention logits scaled by ``attention_multiplier`` and each block's
    output by ``residual_multiplier``."""

    def __init__(self, c: GraniteConfig, i: int):
        super().__init__(c, i)
        self.self_attn.scaling = c.attention_multiplier
        self.residual_multiplier = c.residual_multiplier


def _host_array(array) -> np.ndarray:
    """A loaded weight as a float32 array of bf16 values (a checkpoint hands over torch tensors)."""
    if type(array).__module__.startswith("torch"):
        return from_torch(array)
    return np.asarray(array, dtype=np.float32)


class Granite(CausalLM):
    """Granite on ``config``'s shape and a checkpoint's ``weights``; the untied output head is
    ``lm_head``, every matrix ``(out, in)`` as the checkpoint ships it."""

    config_class = GraniteConfig
    layer_class = GraniteLayer

    def __init__(self, config: GraniteConfig, weights):
        super().__init__(config, weights)
        # The embedding's multiplier as a row every row is multiplied by.
        scale = round_bf16(np.full(config.hidden_size, config.embedding_multiplier, np.float32))
        self.embed_scale = iron.param(scale)
        if config.logits_scaling != 1:
            # The logits' divisor folded into the final norm's loaded weight.
            norm = self.model.norm
            divisor = round_bf16(np.float32(config.logits_scaling))
            norm.weight = iron.param(round_bf16(_host_array(norm.weight.array) / divisor))

    def lookup(self, ids):
        x = super().lookup(ids)
        if self.config.embedding_multiplier == 1:
            return x
        E = self.config.hidden_size
        x = x.reshape(math.prod(x.shape) // E, E)
        return x * self.embed_scale


def shapes(config: DecoderConfig) -> dict[str, tuple[int, ...]]:
    """Each tensor of a Hugging Face Granite checkpoint of ``config``'s shape: Llama's names and
    the untied ``lm_head`` last (tests/applications/granite/reference/test.py:40-44)."""
    from .llama import shapes as llama_shapes

    return llama_shapes(config) | {"lm_head.weight": (config.vocab_size, config.hidden_size)}

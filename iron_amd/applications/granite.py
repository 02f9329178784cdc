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


def _multiplier(default=None):
    """A keyword-only config scalar (keyword-only so it may follow the base class's defaults)."""
    if default is None:
        return dataclasses.field(kw_only=True)
    return dataclasses.field(default=default, kw_only=True)


@dataclasses.dataclass(frozen=True)
class GraniteConfig(DecoderConfig):
    """The shared decoder's config plus the four numbers a Granite ``config.json`` adds."""

    attention_multiplier: float = _multiplier()        # replaces 1/sqrt(head_dim) on the scores
    residual_multiplier: float = _multiplier(1.0)      # on each block's output, ahead of its residual
    embedding_multiplier: float = _multiplier(1.0)     # on the embedding rows
    logits_scaling: float = _multiplier(1.0)           # the logits are DIVIDED by this
    precision: Precision = _multiplier(Precision.HIGH)


class GraniteLayer(DecoderLayer):
    """A Llama layer that hands two of the config's scalars on: the score scale to its attention
    and the residual weight to both of its sums (which the fused GEMVs apply in their epilogue)."""

    def __init__(self, c: GraniteConfig, i: int):
        super().__init__(c, i)
        self.residual_multiplier = c.residual_multiplier
        self.self_attn.scaling = c.attention_multiplier


def _as_float32(weight) -> np.ndarray:
    """float32 values of a weight however the checkpoint delivered it (numpy, or a torch bf16 tensor)."""
    is_torch = type(weight).__module__.split(".")[0] == "torch"
    return from_torch(weight) if is_torch else np.asarray(weight, dtype=np.float32)


class Granite(CausalLM):
    """Granite = the shared decoder + ``GraniteLayer`` + a scaled embedding + scaled logits + an
    untied ``lm_head``.  Neither scale costs a launch of its own at decode time beyond the
    embedding's one rowwise multiply: the logits' divisor is baked into the final norm's gain when
    the weights are loaded."""

    config_class = GraniteConfig
    layer_class = GraniteLayer

    def __init__(self, config: GraniteConfig, weights):
        super().__init__(config, weights)
        width = config.hidden_size
        # a constant row: multiplying every embedding row by it is the config's embedding_multiplier
        self.embed_scale = iron.param(round_bf16(np.full(width, config.embedding_multiplier, dtype=np.float32)))
        if config.logits_scaling != 1:
            final = self.model.norm
            gain = _as_float32(final.weight.array) / round_bf16(np.float32(config.logits_scaling))
            final.weight = iron.param(round_bf16(gain))

    def lookup(self, ids):
        rows = super().lookup(ids)
        if self.config.embedding_multiplier == 1:
            return rows
        width = self.config.hidden_size
        return rows.reshape(math.prod(rows.shape) // width, width) * self.embed_scale


def shapes(config: DecoderConfig) -> dict[str, tuple[int, ...]]:
    """Llama's tensors, then the separate output head a Granite checkpoint ends with
    (tests/applications/granite/reference/test.py:40-44)."""
    from . import llama

    named = llama.shapes(config)
    named["lm_head.weight"] = (config.vocab_size, config.hidden_size)
    return named

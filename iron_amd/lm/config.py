"""The numbers that define a decoder (``DecoderConfig``) and the rotary table they imply
(``rope_angles``).

Fields carry the names of a Hugging Face ``config.json`` wherever that file has the notion, so a
config can be read from and written to one; the interface follows iron/lm/config.py:23-42,184-267.
"""

from __future__ import annotations

import dataclasses
import json
from collections.abc import Callable
from pathlib import Path

import numpy as np

from ..common.declare import Precision

RopeScaling = Callable[[np.ndarray], np.ndarray]

_ACTIVATIONS = ("silu", "gelu_pytorch_tanh", "gelu")


def rope_angles(head_dim: int, context_length: int, rope_theta: float = 500000.0,
                scaling: RopeScaling | None = None) -> np.ndarray:
    """The rotary table: float32 ``(context_length, head_dim)``; column ``2i`` holds
    ``cos(p * f_i)`` and column ``2i + 1`` holds ``sin(p * f_i)`` for position ``p``.

    Precision recipe (it fixes the table bit for bit, so it is part of the contract): the exponent
    ``2i / head_dim`` is float32; ``f_i = theta ** -exponent`` is evaluated in float64, passed through
    ``scaling`` if any, then rounded to float32; ``p * f_i`` is a float32 product; cos and sin are
    taken in float64 and rounded to float32 once.
    """
    pair = np.arange(head_dim // 2 + head_dim % 2, dtype=np.float32) * np.float32(2)
    exponent = (pair / np.float32(head_dim)).astype(np.float64)
    frequency = np.reciprocal(np.power(rope_theta, exponent))
    if scaling is not None:
        frequency = scaling(frequency)
    frequency = frequency.astype(np.float32)
    position = np.arange(context_length, dtype=np.float32)
    phase = (position[:, None] * frequency[None, :]).astype(np.float64)
    table = np.stack((np.cos(phase), np.sin(phase)), axis=-1)
    return table.reshape(context_length, -1)[:, :head_dim].astype(np.float32)


def _required(field: dataclasses.Field) -> bool:
    return field.default is dataclasses.MISSING and field.default_factory is dataclasses.MISSING


@dataclasses.dataclass(frozen=True)
class DecoderConfig:
    """Shape and options of a decoder.  ``max_seq_len`` starts as the checkpoint's native context
    and is usually lowered by the caller (it sizes the KV caches and the rotary table)."""

    vocab_size: int
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    intermediate_size: int
    rope_theta: float | None
    max_seq_len: int
    head_dim: int | None = None
    rope_scaling: RopeScaling | None = None
    eps: float = 1e-6
    precision: Precision = Precision.HIGHEST
    prefill_chunk: int = 2048
    hidden_act: str = "silu"
    tie_word_embeddings: bool = True
    attention_bias: bool = False
    mlp_bias: bool = False
    sliding_window: int | None = None
    # Partial rotary: RoPE turns only the first ``rotary_dim`` columns of each head (None: all of them).
    # Not a config.json field; a model's own config class sets it from whatever its checkpoint calls it.
    rotary_dim: int | None = None

    # field -> its key in config.json when that differs from the field's name.  None marks a field
    # that is this package's own choice: never read from a checkpoint, never written to one.
    JSON = {"eps": "rms_norm_eps", "max_seq_len": "max_position_embeddings", "precision": None,
            "prefill_chunk": None, "rotary_dim": None}

    def __post_init__(self):
        fix = object.__setattr__           # the dataclass is frozen; these two are derived defaults
        if self.head_dim is None:
            fix(self, "head_dim", self.hidden_size // self.num_attention_heads)
        if self.prefill_chunk > self.max_seq_len:
            fix(self, "prefill_chunk", self.max_seq_len)
        if self.rotary_dim is not None and not (0 < self.rotary_dim <= self.head_dim and self.rotary_dim % 16 == 0
                                                and (self.head_dim - self.rotary_dim) % 8 == 0):
            raise ValueError(f"{type(self).__name__}: rotary_dim {self.rotary_dim} of head_dim {self.head_dim}: a "
                             "multiple of 16 that leaves a multiple of 8")
        if self.hidden_act not in _ACTIVATIONS:
            raise ValueError(f"{type(self).__name__}: hidden_act {self.hidden_act!r}: no operator here computes it")

    # -- config.json in and out
    @classmethod
    def _json_key(cls, name: str) -> str | None:
        return cls.JSON[name] if name in cls.JSON else name

    @classmethod
    def from_checkpoint(cls, path):
        """Read ``config.json`` given that file, the checkpoint directory, or any file in it.

        Raises:
            FileNotFoundError: there is no ``config.json`` there.
            ValueError: a field without a default is absent from it.
        """
        where = Path(path)
        if where.name != "config.json":
            where = (where if where.is_dir() else where.parent) / "config.json"
        with open(where) as handle:
            return cls.from_json(json.load(handle), where)

    @classmethod
    def from_json(cls, data: dict, source="config.json"):
        """Build from an already parsed ``config.json``; ``source`` only labels error messages.
        Hugging Face writes ``null`` for options left unset, which reads the same as absent."""
        given, absent = {}, []
        for field in dataclasses.fields(cls):
            key = cls._json_key(field.name)
            if key is None:
                continue
            raw = data.get(key)
            if raw is not None:
                given[field.name] = cls.convert(field.name, raw)
            elif _required(field):
                absent.append(key)
        if absent:
            raise ValueError(f"{source} lacks {absent}")
        return cls(**given)

    @classmethod
    def convert(cls, name: str, value):
        """Hook: a raw ``config.json`` value -> what the field stores.  The base class understands
        only the trivial rotary scaling."""
        if name != "rope_scaling":
            return value
        kind = value.get("rope_type", value.get("type"))
        if kind == "default":
            return None
        raise ValueError(f"rope_scaling {value}: no RoPE table here builds it")

    def to_json(self) -> dict:
        """The inverse of ``from_json``: plain JSON values under ``config.json``'s keys."""
        plain = (bool, int, float, str, tuple, dict)
        out = {}
        for field in dataclasses.fields(self):
            key, value = self._json_key(field.name), getattr(self, field.name)
            if key is None:
                continue
            if dataclasses.is_dataclass(value) and not isinstance(value, type):
                value = dataclasses.asdict(value)
            if isinstance(value, plain):
                out[key] = list(value) if isinstance(value, tuple) else value
        return out

    # -- derived quantities
    @property
    def window(self) -> int | None:
        """Earlier positions a query may see (its own excluded), or None when attention is global or
        the window covers the whole context anyway."""
        span = self.sliding_window
        return None if span is None or span >= self.max_seq_len else span - 1

    @property
    def rope_width(self) -> int:
        """Width of the rotary table: the columns of a head that turn."""
        return self.rotary_dim or self.head_dim

    def angles(self) -> np.ndarray | None:
        """This config's rotary table (a row per position), or None for a model without RoPE."""
        if self.rope_theta is None:
            return None
        return rope_angles(self.rope_width, self.max_seq_len, self.rope_theta, self.rope_scaling)

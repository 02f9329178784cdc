"""A decoder's shape (``DecoderConfig``) and its RoPE table (``rope_angles``).

Field names are a Hugging Face checkpoint's ``config.json``'s where it has one
(iron/lm/config.py:23-42,184-267).
"""

from __future__ import annotations

import dataclasses
import json
from collections.abc import Callable
from pathlib import Path

import numpy as np

from ..common.declare import Precision

RopeScaling = Callable[[np.ndarray], np.ndarray]


def rope_angles(head_dim: int, context_length: int, rope_theta: float = 500000.0,
                scaling: RopeScaling | None = None) -> np.ndarray:
    """Return the RoPE table, ``(context_length, head_dim)`` float32, cos and sin interleaved.

    The frequency and the position are float32, their product float32; each transcendental
    is evaluated in float64 and rounded once.
    """
    exponents = np.arange(0, head_dim, 2, dtype=np.float32) / np.float32(head_dim)
    inv_freq = 1.0 / np.power(rope_theta, exponents.astype(np.float64))
    if scaling is not None:
        inv_freq = scaling(inv_freq)
    inv_freq = inv_freq.astype(np.float32)
    freqs = np.outer(np.arange(context_length, dtype=np.float32), inv_freq)
    angles = np.empty((context_length, head_dim), dtype=np.float32)
    angles[:, ::2] = np.cos(freqs.astype(np.float64))
    angles[:, 1::2] = np.sin(freqs.astype(np.float64))
    return angles


@dataclasses.dataclass(frozen=True)
class DecoderConfig:
    """A decoder's shape. ``max_seq_len`` is the checkpoint's native context unless a caller lowers it."""

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

    # Where a checkpoint's config.json holds a field, where that is not the field's own name; None:
    # nowhere -- a choice of this package, kept at its default by ``from_checkpoint`` and left out
    # by ``to_json`` (iron/lm/config.py:68-183).
    JSON = {"eps": "rms_norm_eps", "max_seq_len": "max_position_embeddings", "precision": None,
            "prefill_chunk": None}

    @classmethod
    def from_checkpoint(cls, path):
        """The fields read from ``path``'s ``config.json``: ``path`` is that file, or a checkpoint's
        directory or one of its files.

        Raises:
            FileNotFoundError: no ``config.json`` is there.
            ValueError: the file lacks a field that has no default.
        """
        path = Path(path)
        if path.name != "config.json":
            path = (path if path.is_dir() else path.parent) / "config.json"
        return cls.from_json(json.loads(path.read_text()), path)

    @classmethod
    def from_json(cls, data: dict, source="config.json"):
        """``from_checkpoint`` on ``data``, a ``config.json`` already parsed; ``source`` names it in an error."""
        kwargs, missing = {}, []
        for f in dataclasses.fields(cls):
            key = cls.JSON.get(f.name, f.name)
            if key is None:
                continue
            value = data.get(key)
            if value is None:  # absent, or Hugging Face's null for an unset option
                if f.default is dataclasses.MISSING and f.default_factory is dataclasses.MISSING:
                    missing.append(key)
                continue
            kwargs[f.name] = cls.convert(f.name, value)
        if missing:
            raise ValueError(f"{source} lacks {missing}")
        return cls(**kwargs)

    @classmethod
    def convert(cls, name: str, value):
        """A ``config.json`` value as the field holds it."""
        if name == "rope_scaling":
            kind = value.get("rope_type", value.get("type"))
            if kind != "default":
                raise ValueError(f"rope_scaling {value}: no RoPE table here builds it")
            return None
        return value

    def to_json(self) -> dict:
        """The fields as ``config.json`` names them: ``from_json``'s inverse."""
        out = {}
        for f in dataclasses.fields(self):
            key = self.JSON.get(f.name, f.name)
            value = getattr(self, f.name)
            if dataclasses.is_dataclass(value) and not isinstance(value, type):
                value = dataclasses.asdict(value)
            if key is None or not isinstance(value, (bool, int, float, str, tuple, dict)):
                continue
            out[key] = list(value) if isinstance(value, tuple) else value
        return out

    def __post_init__(self):
        if self.head_dim is None:
            object.__setattr__(self, "head_dim", self.hidden_size // self.num_attention_heads)
        if self.prefill_chunk > self.max_seq_len:
            object.__setattr__(self, "prefill_chunk", self.max_seq_len)
        if self.hidden_act not in ("silu", "gelu_pytorch_tanh", "gelu"):
            raise ValueError(f"{type(self).__name__}: hidden_act {self.hidden_act!r}: no operator here computes it")

    @property
    def window(self) -> int | None:
        """The positions before a query each layer attends to, ``sliding_window`` less the query's own."""
        if self.sliding_window is None or self.sliding_window >= self.max_seq_len:
            return None
        return self.sliding_window - 1

    @property
    def rope_width(self) -> int:
        return self.head_dim

    def angles(self) -> np.ndarray | None:
        """The RoPE table, a row per position; None with no ``rope_theta``."""
        if self.rope_theta is None:
            return None
        return rope_angles(self.rope_width, self.max_seq_len, self.rope_theta, self.rope_scaling)

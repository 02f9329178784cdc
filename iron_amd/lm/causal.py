"""A decoder-only language model on the GPU, as one graph (iron/lm/causal.py:40-508).

A call with no tensor is a decode step; ``prefill_chunk`` token ``ids`` are a prompt chunk
from ``start``, of which a call runs the first ``rows``.  Both draw the next token on the
device and carry it and ``position + 1`` into the next call.  The decode step is captured
in a HIP graph that carries its own values, so a run of decode steps is a run of replays.
"""

from __future__ import annotations

import dataclasses
import functools
import json
import time
from collections.abc import Iterator
from pathlib import Path
from typing import Any

import numpy as np

from ..common import graph as iron
from ..common.graph import Carried, Scratchpad
from ..operators.copy import Copy
from ..operators.sample import ROW_WORDS, Sample
from .blocks import DecoderLayer, Embedding, Linear, RMSNorm, Rope
from .config import DecoderConfig
from .session import Session


@dataclasses.dataclass(kw_only=True)
class Call:
    """One call's values, built once in ``body`` and read by every memory module
    (``KVCache``, ``Rope``): a prompt chunk's ``rows`` from ``start``, or the decode step's
    one at ``position``."""

    prompt: bool
    start: Any
    rows: Any
    position: Any
    rope_start: Any = None
    ropes: dict = dataclasses.field(default_factory=dict)
    ids: Any = None
    token: Any = None
    embeddings: Any = None


@dataclasses.dataclass
class Stats:
    """What a generation measured: seconds to the first token, tokens per second after it."""

    ttft: float = 0.0
    tokens_per_s: float = 0.0
    tokens: int = 0


class Decoder(iron.Graph):
    """A decoder's modules as a checkpoint's ``model`` names them."""

    def __init__(self, c: DecoderConfig, layer=DecoderLayer):
        self.embed_tokens = Embedding(c.vocab_size, c.hidden_size)
        self.layers = [layer(c, i) for i in range(c.num_hidden_layers)]
        self.norm = RMSNorm(c.hidden_size, c.eps)


class CausalLM(iron.Graph):
    """A decoder on ``config``'s shape: ``model``, ``lm_head`` and ``rotary_emb``."""

    decoder_class = Decoder
    layer_class = DecoderLayer
    #: The config class ``from_checkpoint`` builds from a checkpoint's ``config.json``.
    config_class = DecoderConfig
    checkpoint = None
    tokenizer = None

    @classmethod
    def from_checkpoint(cls, path, *, max_seq_len: int | None = None, **changes):
        """The model of a checkpoint directory's files (``config.json``, ``model.safetensors`` or its
        sharded index, ``tokenizer.json``), not yet loaded (iron/lm/model.py:321-388).

        Args:
            path: the directory (nothing is downloaded here).
            max_seq_len: the longest context served, at most the checkpoint's own.
            changes: other config fields replaced (``prefill_chunk=...``).

        Raises:
            ValueError: ``max_seq_len`` is past the checkpoint's own.
        """
        from .checkpoint import Checkpoint, weights_file
        from .tokenizer import Tokenizer, TokenizerJson

        directory = Path(path)
        if not directory.is_dir():
            raise FileNotFoundError(f"{directory} is not a checkpoint directory (repositories are not downloaded)")
        config = cls.config_class.from_checkpoint(directory)
        if max_seq_len is not None:
            if max_seq_len > config.max_seq_len:
                raise ValueError(f"max_seq_len {max_seq_len} is past the model's {config.max_seq_len}")
            changes["max_seq_len"] = max_seq_len
        if changes:
            config = dataclasses.replace(config, **changes)
        checkpoint = Checkpoint(weights_file(directory))
        # On the device a bf16 tensor goes up as the file holds it; the host stand-in computes on arrays.
        weights = checkpoint.state_dict(as_torch=not issubclass(cls, OnHost))
        if config.tie_word_embeddings:
            weights.pop("lm_head.weight", None)  # some exports repeat the tied matrix
        model = cls(config, weights)
        model.checkpoint = checkpoint
        if (directory / "tokenizer.json").exists():
            settings, jinja = directory / "tokenizer_config.json", directory / "chat_template.jinja"
            found = json.loads(settings.read_text()) if settings.exists() else {}
            template = jinja.read_text() if jinja.exists() else found.get("chat_template")
            b = found.get("bos_token")
            bos_token = (b["content"] if isinstance(b, dict) else b) or ""
            model.tokenizer = Tokenizer(TokenizerJson(directory / "tokenizer.json"), template, bos_token)
        return model

    @classmethod
    def load(cls, path, *, max_seq_len: int | None = None, capture: bool = True, **changes):
        """``from_checkpoint``'s model compiled and loaded, its weights uploaded."""
        model = cls.from_checkpoint(path, max_seq_len=max_seq_len, **changes)
        model.load_versions(capture=capture)
        return model

    @functools.cached_property
    def eos(self) -> set[int]:
        """The tokens generation stops at: the checkpoint's ``eos_token_id``, one or a list, from its
        ``generation_config.json`` or else its ``config.json``; none without either."""
        if self.checkpoint is None:
            return set()
        directory = Path(self.checkpoint.path).parent
        for name in ("generation_config.json", "config.json"):
            file = directory / name
            if file.exists():
                eos = json.loads(file.read_text()).get("eos_token_id")
                if eos is not None:
                    return set(eos) if isinstance(eos, list) else {eos}
        return set()

    #: The most candidates a draw on the device weighs (``Sampler.rows`` refuses a larger top-k).
    k_max = 64

    def __init__(self, config: DecoderConfig, weights):
        self.config = config
        self.rotary_emb = None if config.rope_theta is None else Rope(config)
        # Zero until the host writes draws: a row of zeros is greedy.
        self.draws = iron.state((config.max_seq_len, ROW_WORDS), np.int32)
        self.drawn = iron.state((config.max_seq_len,), np.int32)
        self.sampled = False  # the draw rows hold a sampler's, not zeros
        self.prompt_chunk = None
        self.decode_step = None
        self.holder = None
        self.session = Session(self)
        self.stats = Stats()
        self.model = self.decoder_class(config, self.layer_class)
        for layer in self.model.layers:
            layer.rope = self.rotary_emb
        self.lm_head = Linear(config.hidden_size, config.vocab_size, False, precision=config.precision)
        if config.tie_word_embeddings:
            self.lm_head.weight = self.model.embed_tokens.weight
        self.load_state_dict(weights)
        self.layers = self.model.layers

    @property
    def recurrent(self) -> list:
        """The states that restart only at some positions: the layers' ring caches."""
        rings = {id(l.cache): l.cache for l in self.layers if getattr(l.cache, "ring", None) is not None}
        return list(rings.values())

    def layer(self, call, i: int, w, x):
        """Layer ``i``, ``w``, on ``x``: a model whose layers take more than the call says what."""
        return w(x, call)

    def head(self, x):
        """The final norm, then the output head (the embedding, if tied)."""
        return self.lm_head(self.model.norm(x))

    def lookup(self, ids):
        return self.model.embed_tokens(ids)

    def body(self, ids=None, *, token: Carried[np.int32], position: Carried[np.int32],
             start: Scratchpad[np.int32] = np.int32(0), rows: Scratchpad[np.int32] = np.int32(1),
             rope_start: Scratchpad[np.int32] = np.int32(0)):
        prompt = ids is not None
        call = Call(prompt=prompt, start=start if prompt else position, rows=rows, position=position,
                    rope_start=rope_start, ids=ids[:rows] if prompt else token, token=token)
        if prompt:
            return self.forward(self.lookup(call.ids), call)
        return self.forward(self.lookup(token).reshape(1, self.config.hidden_size), call)

    def forward(self, x, call: Call):
        """The layers, the head and the draw over ``x``, the rows ``call`` runs."""
        c = self.config
        call.embeddings = x
        for rope in (layer.rope for layer in self.layers):
            if rope is not None and id(rope) not in call.ropes:
                call.ropes[id(rope)] = rope.rows(call)
        for i, layer in enumerate(self.layers):
            x = self.layer(call, i, layer, x)
        if call.prompt:
            x = Copy.step(x[call.rows - 1]).reshape(1, c.hidden_size)  # the last row's logits alone
        return self.draw(self.head(x), call)

    def draw(self, logits, call: Call):
        """``logits`` and the token drawn from them on the device, carried with the next position."""
        c = self.config
        _, drawn = Sample.step(logits.reshape(c.vocab_size), self.draws, self.drawn,
                               row=call.position * ROW_WORDS, at=call.position, drawable=c.vocab_size,
                               k_max=self.k_max)
        return logits, iron.carry(token=drawn, position=call.position + 1)

    # -- versions ------------------------------------------------------------
    def shapes(self) -> list[dict]:
        """The input shapes of each version: the decode step's (none), then the prompt chunk's ids."""
        return [{}, dict(ids=((self.config.prefill_chunk,), np.int32))]

    def load_versions(self, *, capture: bool = True, check: bool = False, fuse: bool = True) -> None:
        """Compile the decode step and the prompt chunk into one arena and load them.

        ``fuse``: launch the decode step's runs of one-row steps as fused kernels.
        """
        decode_shapes, prompt_shapes = self.shapes()
        try:
            decode = self.compile(capture=capture, check=check, fuse=fuse, **decode_shapes)
            prompt = self.compile(capture=False, check=check, fuse=fuse, **prompt_shapes)
            decode.load()
            prompt.load()
        except Exception:
            self.release()
            raise
        self.use(decode, prompt)

    def use(self, decode, prompt) -> None:
        self.decode_step, self.prompt_chunk = decode, prompt
        self.holder = None

    def release(self) -> None:
        self.decode_step = self.prompt_chunk = None
        super().release()

    def __call__(self, ids=None, **values):
        """One call of the prompt version or else the decode step."""
        if iron.graph_recorder.get() is not None:
            return super().__call__(ids, **values)
        if self.decode_step is None:
            raise RuntimeError(f"{type(self).__name__}: load_versions() first")
        if ids is None:
            return self.decode_step(**values)
        return self.prompt_chunk(ids, **values)

    def logits(self, tokens) -> np.ndarray:
        """The logits after the last of ``tokens``, the whole history (``Session.logits``)."""
        return self.session.logits(tokens)

    def generate(self, prompt, max_tokens: int, sampler=None):
        """Up to ``max_tokens`` tokens drawn on the device after ``prompt``, stopping after an
        end-of-sequence token; fills ``stats``.  Token ids in, token ids out; a text (or a chat's
        list of messages) in, the text drawn out (needs the checkpoint's tokenizer).  ``sampler``:
        how each is drawn (``generation.Sampler``); None is greedy (iron/lm/model.py:506-545)."""
        if _is_text(prompt):
            drawn = [t for t in self.stream(prompt, max_tokens, sampler) if t not in self.eos]
            return self.tokenizer.decode(drawn)
        return list(self.stream(prompt, max_tokens, sampler))

    def _ids(self, prompt):
        if not _is_text(prompt):
            return prompt
        if self.tokenizer is None:
            raise ValueError(f"{type(self).__name__}: a text prompt takes the checkpoint's tokenizer; none is loaded")
        return self.tokenizer(prompt) if isinstance(prompt, str) else self.tokenizer.chat(prompt)

    def stream(self, prompt, max_tokens: int, sampler=None) -> Iterator[int]:
        tokens = self._ids(prompt)
        t0 = time.perf_counter()
        first = None
        n = 0
        for token in self.session.draw(tokens, max_tokens, sampler):
            n += 1
            if first is None:
                first = time.perf_counter()
            yield token
            if token in self.eos:
                break
        end = time.perf_counter()
        self.stats = Stats(ttft=(first or end) - t0,
                           tokens_per_s=(n - 1) / (end - first) if n > 1 and end > first else 0.0, tokens=n)


def _is_text(prompt) -> bool:
    """A string, or a chat: a list of ``{"role": ..., "content": ...}`` messages."""
    return isinstance(prompt, str) or (isinstance(prompt, list) and bool(prompt) and isinstance(prompt[0], dict))


class _HostOutput:
    def __init__(self, array):
        self.array = array

    def numpy(self):
        return self.array


class _HostVersion:
    """A version stood in by the graph's host reference: same call, numpy underneath."""

    captured = False

    def __init__(self, graph, takes_ids: bool):
        self.graph, self.takes_ids = graph, takes_ids

    def __call__(self, *tensors, **values):
        outs, carried = iron.Graph.reference(self.graph, *tensors, **values)
        return (*(_HostOutput(o) for o in outs), iron.Carry(carried))

    def write(self, resident, array) -> None:
        resident.host = np.array(array).reshape(-1)

    def read(self, resident) -> np.ndarray:
        host = getattr(resident, "host", None)
        return np.zeros(resident.shape, np.int32) if host is None else host.reshape(resident.shape)


class OnHost:
    """Mix-in: the model with its compiled versions replaced by ``Graph.reference``, which runs
    the graph operator by operator on host arrays with the caches as state -- the fake backend
    of the device-free model tests (iron/lm/model.py:667-695).  Needs a registered CPU
    reference for every operator (the test oracle)."""

    def load_versions(self, **_):
        self.use(_HostVersion(self, False), _HostVersion(self, True))

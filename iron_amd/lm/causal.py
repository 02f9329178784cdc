"""A decoder-only language model as ONE graph with two compiled versions sharing an arena.

Interface of the reference's iron/lm/causal.py:40-508 and iron/lm/model.py:321-597.  ``body`` is
recorded twice: without ``ids`` it is the *decode step* (one token at ``position``), with
``prefill_chunk`` ids it is a *prompt chunk* (``rows`` tokens from ``start``).  Either version ends
by drawing the next token on the device and carrying ``token`` / ``position + 1`` forward.  On the
GPU the decode step is captured in a HIP graph whose tail re-derives its own per-call words, so
generating N tokens is N replays with no host round trip between them.
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
    """The per-call quantities of one recording, gathered once so that every stateful module
    (caches, rotary tables) reads the same ones.  ``prompt`` tells the two versions apart; for a
    decode step ``start`` is the position and ``rows`` is 1.  ``ropes`` memoises each rotary
    table's rows for this call by table identity; ``embeddings`` is the layers' input, kept for
    models whose layers look back at it."""

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
    """Timing of the last ``generate`` / ``stream``: time to first token (s), decode rate after it
    (tokens/s), and how many tokens came out."""

    ttft: float = 0.0
    tokens_per_s: float = 0.0
    tokens: int = 0


class Decoder(iron.Graph):
    """The trunk under a checkpoint's ``model.`` prefix: embedding, layers, final norm."""

    def __init__(self, c: DecoderConfig, layer=DecoderLayer):
        self.embed_tokens = Embedding(c.vocab_size, c.hidden_size)
        self.layers = [layer(c, index) for index in range(c.num_hidden_layers)]
        self.norm = RMSNorm(c.hidden_size, c.eps)


def _read_json(path: Path) -> dict:
    return json.loads(path.read_text()) if path.exists() else {}


class CausalLM(iron.Graph):
    """``model`` (the trunk), ``lm_head`` (tied to the embedding unless the config says otherwise)
    and ``rotary_emb``.  Subclasses vary it through ``config_class`` / ``layer_class`` /
    ``decoder_class`` and the hooks ``lookup``, ``layer``, ``head``."""

    decoder_class = Decoder
    layer_class = DecoderLayer
    config_class = DecoderConfig      # what from_checkpoint parses config.json into
    checkpoint = None
    tokenizer = None
    k_max = 64                        # candidates a device draw can weigh; Sampler.rows refuses a larger top-k

    # ------------------------------------------------------------------ construction
    def __init__(self, config: DecoderConfig, weights):
        self.config = config
        self.rotary_emb = Rope(config) if config.rope_theta is not None else None
        rows = config.max_seq_len
        self.draws = iron.state((rows, ROW_WORDS), np.int32)   # a draw row per position; all-zero = greedy
        self.drawn = iron.state((rows,), np.int32)             # the device's record of what it drew where
        self.sampled = False          # whether `draws` currently holds a sampler's rows
        self.decode_step = self.prompt_chunk = None
        self.holder = None            # the Session whose tokens the caches hold
        self.session = Session(self)
        self.stats = Stats()
        self.model = self.decoder_class(config, self.layer_class)
        self.layers = self.model.layers
        for block in self.layers:
            block.rope = self.rotary_emb
        self.lm_head = Linear(config.hidden_size, config.vocab_size, False, precision=config.precision)
        if config.tie_word_embeddings:
            self.lm_head.weight = self.model.embed_tokens.weight
        self.load_state_dict(weights)

    @classmethod
    def from_checkpoint(cls, path, *, max_seq_len: int | None = None, **changes):
        """Build (not yet compile) the model described by a local checkpoint directory:
        ``config.json``, ``model.safetensors`` or a shard index, optionally ``tokenizer.json`` with
        ``tokenizer_config.json`` / ``chat_template.jinja`` (iron/lm/model.py:321-388).  Nothing is
        fetched from anywhere.

        Args:
            max_seq_len: context to serve; may only shrink the checkpoint's own.
            changes: further config overrides, e.g. ``prefill_chunk=512``.

        Raises:
            FileNotFoundError: ``path`` is not a directory.
            ValueError: ``max_seq_len`` exceeds what the checkpoint supports.
        """
        from .checkpoint import Checkpoint, weights_file
        from .tokenizer import Tokenizer, TokenizerJson

        folder = Path(path)
        if not folder.is_dir():
            raise FileNotFoundError(f"{folder} is not a checkpoint directory (repositories are not downloaded)")
        config = cls.config_class.from_checkpoint(folder)
        if max_seq_len is not None and max_seq_len > config.max_seq_len:
            raise ValueError(f"max_seq_len {max_seq_len} is past the model's {config.max_seq_len}")
        overrides = dict(changes) if max_seq_len is None else {**changes, "max_seq_len": max_seq_len}
        if overrides:
            config = dataclasses.replace(config, **overrides)
        checkpoint = Checkpoint(weights_file(folder))
        # The GPU takes bf16 exactly as stored (torch views of the mapped file); only the host
        # stand-in wants widened arrays to compute on.
        weights = checkpoint.state_dict(as_torch=not issubclass(cls, OnHost))
        if config.tie_word_embeddings and "lm_head.weight" in weights:
            del weights["lm_head.weight"]       # some exporters write the tied matrix twice
        model = cls(config, weights)
        model.checkpoint = checkpoint
        vocabulary = folder / "tokenizer.json"
        if vocabulary.exists():
            settings = _read_json(folder / "tokenizer_config.json")
            template_file = folder / "chat_template.jinja"
            template = template_file.read_text() if template_file.exists() else settings.get("chat_template")
            bos = settings.get("bos_token")
            if isinstance(bos, dict):           # {"content": "<s>", ...} in older configs
                bos = bos.get("content")
            model.tokenizer = Tokenizer(TokenizerJson(vocabulary), template, bos or "")
        return model

    @classmethod
    def load(cls, path, *, max_seq_len: int | None = None, capture: bool = True, **changes):
        """``from_checkpoint`` followed by ``load_versions``: ready to generate."""
        model = cls.from_checkpoint(path, max_seq_len=max_seq_len, **changes)
        model.load_versions(capture=capture)
        return model

    @functools.cached_property
    def eos(self) -> set[int]:
        """Token ids that end a generation: ``eos_token_id`` (a number or a list) from the
        checkpoint's ``generation_config.json``, failing that its ``config.json``; empty for a model
        built from arrays."""
        if self.checkpoint is None:
            return set()
        folder = Path(self.checkpoint.path).parent
        for name in ("generation_config.json", "config.json"):
            declared = _read_json(folder / name).get("eos_token_id")
            if declared is not None:
                return set(declared) if isinstance(declared, list) else {declared}
        return set()

    @property
    def recurrent(self) -> list:
        """State that cannot be rewound to an arbitrary position -- the ring caches -- each once even
        where layers share it.  ``Session.resume`` asks these where a run may restart."""
        seen: dict[int, Any] = {}
        for block in self.layers:
            if getattr(block.cache, "ring", None) is not None:
                seen.setdefault(id(block.cache), block.cache)
        return list(seen.values())

    # ------------------------------------------------------------------ the recorded body
    def lookup(self, ids):
        """Hook: token ids -> embedding rows."""
        return self.model.embed_tokens(ids)

    def layer(self, call, i: int, w, x):
        """Hook: apply layer ``i`` (module ``w``) to ``x``; override where layers take extra inputs."""
        return w(x, call)

    def head(self, x):
        """Hook: final norm and output projection."""
        return self.lm_head(self.model.norm(x))

    def body(self, ids=None, *, token: Carried[np.int32], position: Carried[np.int32],
             start: Scratchpad[np.int32] = np.int32(0), rows: Scratchpad[np.int32] = np.int32(1),
             rope_start: Scratchpad[np.int32] = np.int32(0)):
        if ids is None:
            call = Call(prompt=False, start=position, rows=rows, position=position, rope_start=rope_start,
                        ids=token, token=token)
            x = self.lookup(token).reshape(1, self.config.hidden_size)
        else:
            call = Call(prompt=True, start=start, rows=rows, position=position, rope_start=rope_start,
                        ids=ids[:rows], token=token)
            x = self.lookup(call.ids)
        return self.forward(x, call)

    def forward(self, x, call: Call):
        """Embeddings ``x`` through the layers, the head and the draw."""
        call.embeddings = x
        for block in self.layers:          # each distinct rotary table copies its rows once per call
            table = block.rope
            if table is not None and id(table) not in call.ropes:
                call.ropes[id(table)] = table.rows(call)
        for index, block in enumerate(self.layers):
            x = self.layer(call, index, block, x)
        if call.prompt:
            # only the chunk's last real row feeds the head
            x = Copy.step(x[call.rows - 1]).reshape(1, self.config.hidden_size)
        return self.draw(self.head(x), call)

    def draw(self, logits, call: Call):
        """Draw from ``logits`` by this position's draw row; returns the logits and the carry."""
        vocab = self.config.vocab_size
        _, token = Sample.step(logits.reshape(vocab), self.draws, self.drawn, row=call.position * ROW_WORDS,
                               at=call.position, drawable=vocab, k_max=self.k_max)
        return logits, iron.carry(token=token, position=call.position + 1)

    # ------------------------------------------------------------------ versions
    def shapes(self) -> list[dict]:
        """Input shapes per version: ``[decode step (no tensor), prompt chunk (ids)]``."""
        return [{}, {"ids": ((self.config.prefill_chunk,), np.int32)}]

    def load_versions(self, *, capture: bool = True, check: bool = False, fuse: bool = True) -> None:
        """Compile both versions into the shared arena, upload the weights, capture each as a HIP
        graph (the prompt chunk's ids are copied into its arena slot and its per-call words
        rewritten before every replay).  ``fuse=False`` launches every recorded step on its own
        (what ``check=True`` implies); ``capture=False`` keeps both versions eager."""
        for_decode, for_prompt = self.shapes()
        try:
            decode = self.compile(capture=capture, check=check, fuse=fuse, **for_decode)
            prompt = self.compile(capture=capture, check=check, fuse=fuse, **for_prompt)
            for version in (decode, prompt):
                version.load()
        except Exception:
            self.release()
            raise
        self.use(decode, prompt)

    def use(self, decode, prompt) -> None:
        """Adopt two loaded versions; whatever the caches held belongs to nobody now."""
        self.decode_step, self.prompt_chunk, self.holder = decode, prompt, None

    def release(self) -> None:
        self.decode_step = self.prompt_chunk = None
        super().release()

    def __call__(self, ids=None, **values):
        """Inside a recording: record the body.  Otherwise run a loaded version -- the prompt chunk
        when ``ids`` are given, else the decode step."""
        if iron.graph_recorder.get() is not None:
            return super().__call__(ids, **values)
        if self.decode_step is None:
            raise RuntimeError(f"{type(self).__name__}: load_versions() first")
        return self.decode_step(**values) if ids is None else self.prompt_chunk(ids, **values)

    # ------------------------------------------------------------------ use
    def logits(self, tokens) -> np.ndarray:
        """Logits after the last of ``tokens`` (see ``Session.logits``)."""
        return self.session.logits(tokens)

    def _prompt_ids(self, prompt):
        if not _is_text(prompt):
            return prompt
        if self.tokenizer is None:
            raise ValueError(f"{type(self).__name__}: a text prompt takes the checkpoint's tokenizer; none is loaded")
        return self.tokenizer.chat(prompt) if isinstance(prompt, list) else self.tokenizer(prompt)

    def stream(self, prompt, max_tokens: int, sampler=None) -> Iterator[int]:
        """Yield drawn token ids one by one, stopping after an end-of-sequence id; records ``stats``."""
        ids = self._prompt_ids(prompt)
        began = time.perf_counter()
        first_at, count = None, 0
        for token in self.session.draw(ids, max_tokens, sampler):
            now = time.perf_counter()
            first_at = now if first_at is None else first_at
            count += 1
            yield token
            if token in self.eos:
                break
        ended = time.perf_counter()
        first_at = ended if first_at is None else first_at
        decoding = ended - first_at
        rate = (count - 1) / decoding if count > 1 and decoding > 0 else 0.0
        self.stats = Stats(ttft=first_at - began, tokens_per_s=rate, tokens=count)

    def generate(self, prompt, max_tokens: int, sampler=None):
        """Generate up to ``max_tokens`` tokens on the device (iron/lm/model.py:506-545).  Ids in, ids
        out (the end-of-sequence id included if one was drawn).  A string, or a chat as a list of
        ``{"role", "content"}`` messages, goes through the checkpoint's tokenizer and comes back as
        text without end-of-sequence tokens.  ``sampler=None`` draws greedily."""
        tokens = list(self.stream(prompt, max_tokens, sampler))    # refuses a text prompt without a tokenizer
        if not _is_text(prompt):
            return tokens
        return self.tokenizer.decode([t for t in tokens if t not in self.eos])


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

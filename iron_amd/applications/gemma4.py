"""The text decoder of Gemma 4 (interface of iron/applications/gemma4/model.py:42-246).

What sets it apart from the plain decoder, and where each piece lives:

* layers are "sliding_attention" or "full_attention" by ``layer_types``.  Global layers have wider
  heads (``global_head_dim``) and their own rotary table, of which only the first
  ``partial_rotary_factor`` of the pairs turn -- the rest get frequency 0, i.e. the identity;
* q, k and v are RMS-normed per head and the scores are not scaled (``Gemma4Layer``);
* each block's output is normed before it joins the residual (``SandwichLayer``);
* the last ``num_kv_shared_layers`` layers own no cache: they read the cache of the last earlier
  layer of their kind, and may have a feed-forward twice as wide;
* every layer adds a "per-layer input": the token's row of a per-layer table plus a projection of
  the embeddings, gated into the hidden state (``PleLayer``);
* the logits may be soft-capped with a tanh.

Vision and audio towers are out of scope; a multimodal checkpoint's language model loads from the
tensors under ``model.language_model``.
"""

from __future__ import annotations

import dataclasses

import numpy as np

from .. import functional as F
from ..bf16 import from_torch, round_bf16
from ..common import graph as iron
from ..common.declare import Precision
from ..lm import CausalLM, DecoderConfig
from ..lm.blocks import Attention, Embedding, GatedMLP, KVCache, Linear, PleLayer, RMSNorm, Rope
from ..lm.causal import Decoder
from ..operators.copy import Copy
from ..operators.tanh import Tanh

PREFIX = "model.language_model."

_GLOBAL, _SLIDING = "full_attention", "sliding_attention"


def _walk(tree, dotted: str):
    """``tree["a"]["b"]`` for ``"a.b"``, or None as soon as a level is missing."""
    node = tree
    for part in dotted.split("."):
        node = node.get(part) if isinstance(node, dict) else None
        if node is None:
            return None
    return node


def _kw(default=dataclasses.MISSING):
    return dataclasses.field(kw_only=True) if default is dataclasses.MISSING else dataclasses.field(default=default, kw_only=True)


@dataclasses.dataclass(frozen=True)
class Gemma4Config(DecoderConfig):
    """The decoder's config as a Gemma 4 ``config.json`` spells it: most fields sit under
    ``text_config`` (some nested deeper), the multimodal placeholder ids at the top level."""

    precision: Precision = _kw(Precision.MEDIUM)
    hidden_act: str = "gelu_pytorch_tanh"
    layer_types: tuple[str, ...] = _kw()
    global_head_dim: int = _kw(512)
    global_rope_theta: float = _kw(1000000.0)
    partial_rotary_factor: float = _kw(0.25)
    num_kv_shared_layers: int = _kw(0)
    use_double_wide_mlp: bool = _kw(False)
    ple_dim: int = _kw(256)
    final_logit_softcapping: float | None = _kw(None)
    # Ids that stand for image / audio / video soft tokens.  Without towers they can only be treated
    # as padding by the per-layer table, which is what the full model does with them too.
    pad_token_id: int = _kw(0)
    image_token_id: int | None = _kw(None)
    audio_token_id: int | None = _kw(None)
    video_token_id: int | None = _kw(None)

    # field -> where config.json keeps it, relative to text_config; "/" in front = top level instead
    PATHS = {
        "eps": "rms_norm_eps", "max_seq_len": "max_position_embeddings", "hidden_act": "hidden_activation",
        "rope_theta": "rope_parameters.sliding_attention.rope_theta",
        "global_rope_theta": "rope_parameters.full_attention.rope_theta",
        "partial_rotary_factor": "rope_parameters.full_attention.partial_rotary_factor",
        "ple_dim": "hidden_size_per_layer_input",
        "image_token_id": "/image_token_id", "audio_token_id": "/audio_token_id", "video_token_id": "/video_token_id",
    }
    NOT_JSON = ("precision", "prefill_chunk", "rope_scaling")     # this package's own knobs

    @classmethod
    def _unsupported(cls, text: dict) -> str | None:
        """The first thing ``text_config`` asks for that this decoder does not implement, if any."""
        for flag in ("attention_k_eq_v", "enable_moe_block", "attn_logit_softcapping"):
            if text.get(flag):
                return f"{flag} {text[flag]!r}"
        # "vision" limits bidirectional attention to image tokens, of which text has none
        both_ways = text.get("use_bidirectional_attention")
        if both_ways not in (None, False, "vision"):
            return f"bidirectional attention {both_ways!r}"
        vocab = text.get("vocab_size")
        table_vocab = text.get("vocab_size_per_layer_input", vocab)
        if table_vocab != vocab:
            return f"vocab_size_per_layer_input {table_vocab} other than vocab_size {vocab}"
        ropes = text.get("rope_parameters", {})
        for kind, expected in ((_SLIDING, "default"), (_GLOBAL, "proportional")):
            declared = ropes.get(kind, {}).get("rope_type", expected)
            if declared != expected:
                return f"{kind} RoPE {declared!r}"
        return None

    @classmethod
    def from_json(cls, data: dict, source="config.json") -> "Gemma4Config":
        """Parse a ``config.json`` (iron/applications/gemma4/model.py:89-125).

        Raises:
            ValueError: it asks for a variant not built here (keys tied to values, experts, capped
                attention scores, bidirectional text, a per-layer vocabulary of its own, other RoPE
                kinds), or a field without a default is missing.
        """
        text = dict(data.get("text_config", {}))
        problem = cls._unsupported(text)
        if problem is not None:
            raise ValueError(f"{source}: {problem} is not built here")
        found, absent = {}, []
        for field in dataclasses.fields(cls):
            if field.name in cls.NOT_JSON:
                continue
            where = cls.PATHS.get(field.name, field.name)
            value = _walk(data, where[1:]) if where[0] == "/" else _walk(text, where)
            if value is not None:
                found[field.name] = tuple(value) if field.name == "layer_types" else value
            elif field.default is dataclasses.MISSING and field.default_factory is dataclasses.MISSING:
                absent.append(where)
        if absent:
            raise ValueError(f"{source} lacks {absent}")
        return cls(**found)

    def to_json(self) -> dict:
        """Back to ``config.json``'s layout: ``from_json(to_json())`` reproduces the config."""
        document: dict = {"text_config": {}}
        for field in dataclasses.fields(self):
            value = getattr(self, field.name)
            if value is None or field.name in self.NOT_JSON:
                continue
            where = self.PATHS.get(field.name, field.name)
            scope = document if where[0] == "/" else document["text_config"]
            keys = where.lstrip("/").split(".")
            for key in keys[:-1]:
                scope = scope.setdefault(key, {})
            scope[keys[-1]] = list(value) if isinstance(value, tuple) else value
        return document

    def full(self, i: int) -> bool:
        """True for a global ("full_attention") layer."""
        return self.layer_types[i] == _GLOBAL

    def owner(self, i: int) -> int:
        """Index of the layer whose KV cache layer ``i`` reads: itself, unless ``i`` is one of the
        trailing shared layers -- then the last non-shared layer of the same kind.

        Raises:
            ValueError: a shared layer with no earlier layer of its kind.
        """
        own_caches = self.num_hidden_layers - self.num_kv_shared_layers
        if i < own_caches:
            return i
        for j in range(own_caches - 1, -1, -1):
            if self.full(j) == self.full(i):
                return j
        raise ValueError(f"Gemma4Config: shared layer {i} has no earlier layer of its kind")


class Gemma4Decoder(Decoder):
    """The trunk plus what the per-layer inputs need: one wide token table (all layers' columns side
    by side, as the checkpoint stores it), the projection of the embeddings, and its norm."""

    def __init__(self, c: Gemma4Config, layer):
        super().__init__(c, layer)
        all_layers = c.num_hidden_layers * c.ple_dim
        # only a loading vehicle: split into per-layer tables and dropped in load_state_dict
        self.embed_tokens_per_layer = Embedding(c.vocab_size, all_layers)
        self.per_layer_model_projection = Linear(c.hidden_size, all_layers, False, precision=c.precision)
        self.per_layer_projection_norm = RMSNorm(c.ple_dim, c.eps)


class Gemma4Layer(PleLayer):
    """One Gemma 4 layer: per-head norms on q, k, v; scores used as they are (scale 1); global
    layers with their own head width over the whole context, sliding ones within the window; a
    shared layer optionally with the double-width feed-forward."""

    def __init__(self, c: Gemma4Config, i: int):
        is_global, shared = c.full(i), c.owner(i) != i
        head_config = dataclasses.replace(c, head_dim=c.global_head_dim) if is_global else c
        wide_mlp = None
        if shared and c.use_double_wide_mlp:
            wide_mlp = GatedMLP(dataclasses.replace(c, intermediate_size=2 * c.intermediate_size))
        cache = KVCache(head_config, None if is_global else c.window)
        super().__init__(c, i, Attention(head_config, i, norms="qkv"), wide_mlp, cache)
        self.self_attn.scaling = 1.0


def _as_float32(weight) -> np.ndarray:
    """float32 values of a loaded weight (numpy, or a torch bf16 tensor from a checkpoint)."""
    if type(weight).__module__.split(".")[0] == "torch":
        return from_torch(weight)
    return np.asarray(weight, dtype=np.float32)


class _StillPairs:
    """The "proportional" RoPE of global layers as a frequency scaling: pairs from ``turned`` on get
    frequency 0 and therefore never rotate."""

    def __init__(self, turned: int):
        self.turned = turned

    def __call__(self, inv_freq: np.ndarray) -> np.ndarray:
        keep = np.arange(inv_freq.size) < self.turned
        return np.where(keep, inv_freq, 0)


def _drop_kv(attention) -> None:
    attention.k_proj = attention.v_proj = attention.k_norm = None


class Gemma4(CausalLM):
    """Gemma 4's language model from a config and a checkpoint's tensors by name (those under
    ``model.language_model`` are used, plus an untied ``lm_head`` if present; towers are ignored)."""

    config_class = Gemma4Config
    decoder_class = Gemma4Decoder
    layer_class = Gemma4Layer

    def __init__(self, config: Gemma4Config, weights):
        own = {"model." + name.removeprefix(PREFIX): tensor for name, tensor in weights.items()
               if name.startswith(PREFIX)}
        if "lm_head.weight" in weights:
            own["lm_head.weight"] = weights["lm_head.weight"]
        super().__init__(config, own)
        c = config
        turning_pairs = int(c.partial_rotary_factor * c.global_head_dim // 2)
        global_rope = Rope(dataclasses.replace(c, head_dim=c.global_head_dim, rope_theta=c.global_rope_theta,
                                               rope_scaling=_StillPairs(turning_pairs)))
        for i, block in enumerate(self.layers):
            if c.full(i):
                block.rope = global_rope
            source = c.owner(i)
            if source != i:
                _drop_kv(block.self_attn)
                block.cache = self.layers[source].cache

    def load_state_dict(self, tree, *, path: str = "") -> None:
        c, trunk = self.config, self.model
        # Checkpoints differ on whether shared layers still carry k/v weights they never use.  If
        # they do, load them (they are dropped when the caches are wired up); if not, do not ask.
        for i, block in enumerate(trunk.layers):
            unused = c.owner(i) != i
            if unused and f"{path}model.layers.{i}.self_attn.k_proj.weight" not in tree:
                _drop_kv(block.self_attn)
        super().load_state_dict(tree, path=path)
        width, hidden = c.ple_dim, c.hidden_size
        gain = round_bf16(np.float32(np.sqrt(width)))
        wide_table = _as_float32(trunk.embed_tokens_per_layer.weight.array)
        soft_tokens = [t for t in (c.image_token_id, c.audio_token_id, c.video_token_id) if t is not None]
        for i, block in enumerate(trunk.layers):
            # this layer's columns, pre-scaled and contiguous, so a call gathers one row per token
            table = wide_table[:, i * width : (i + 1) * width] * gain
            table[soft_tokens] = table[c.pad_token_id]
            block.per_layer_embedding = iron.param(round_bf16(table))
            # layer_scalar as a constant row the layer's output is multiplied by
            scalar = _as_float32(block.layer_scalar.array)[0]
            block.scale = iron.param(round_bf16(np.full(hidden, scalar, dtype=np.float32)))
        trunk.embed_tokens_per_layer = None

    def lookup(self, ids):
        """Embedding rows times sqrt(hidden_size) (recorded as a multiply by a constant row)."""
        return super().lookup(ids) * float(np.sqrt(self.config.hidden_size))

    def layer(self, call, i, w, x):
        """Layer ``i`` with its per-layer input: (projection of the embeddings, normed, plus the
        token's table row) / sqrt(2)."""
        c, trunk = self.config, self.model
        width = c.ple_dim
        columns = trunk.per_layer_model_projection.weight[i * width : (i + 1) * width]
        projected = F.linear(call.embeddings, columns, precision=c.precision)
        rows = call.embeddings.elements // c.hidden_size
        # The checkpoint's projection carries a factor hidden_size ** -0.5.  Since
        # RMSNorm(s * y, eps) is RMSNorm(y, eps / s ** 2), it moves into the epsilon for free.
        projected = F.rms_norm(projected.reshape(rows, width), (width,), trunk.per_layer_projection_norm.weight,
                               c.eps * c.hidden_size)
        token = Copy.step(iron.weight(w.per_layer_embedding)[call.ids])
        return w(x, call, (projected + token.reshape(projected.shape)) * 2**-0.5)

    def head(self, x):
        """Logits, soft-capped as ``cap * tanh(logits / cap)`` when the config sets a cap."""
        logits = super().head(x)
        cap = self.config.final_logit_softcapping
        if cap is None:
            return logits
        return Tanh.step(logits * (1 / cap)) * cap


# per-layer tensors in the order the reference's toy draws them
# (tests/applications/gemma4/reference/test.py:60-108); letters: E hidden, Q q width, K kv width,
# D head width, M feed-forward width, P per-layer width
_LAYER_TENSORS = (
    ("self_attn.q_proj.weight", "QE"), ("self_attn.o_proj.weight", "EQ"), ("self_attn.q_norm.weight", "D"),
    ("mlp.gate_proj.weight", "ME"), ("mlp.up_proj.weight", "ME"), ("mlp.down_proj.weight", "EM"),
    ("per_layer_input_gate.weight", "PE"), ("per_layer_projection.weight", "EP"), ("layer_scalar", "1"),
    # shipped for shared layers as well, though those never read them
    ("self_attn.k_proj.weight", "KE"), ("self_attn.v_proj.weight", "KE"), ("self_attn.k_norm.weight", "D"),
    ("input_layernorm.weight", "E"), ("post_attention_layernorm.weight", "E"),
    ("pre_feedforward_layernorm.weight", "E"), ("post_feedforward_layernorm.weight", "E"),
    ("post_per_layer_input_norm.weight", "E"),
)


def shapes(config: Gemma4Config) -> dict[str, tuple[int, ...]]:
    """Name -> shape for the language model's tensors of a Hugging Face Gemma 4 checkpoint of this
    config, in the order a seeded draw of the reference's toy follows."""
    c = config
    layers, hidden, width, vocab = c.num_hidden_layers, c.hidden_size, c.ple_dim, c.vocab_size
    root = PREFIX.rstrip(".")
    named = {
        f"{root}.embed_tokens.weight": (vocab, hidden),
        f"{root}.norm.weight": (hidden,),
        f"{root}.embed_tokens_per_layer.weight": (vocab, layers * width),
        f"{root}.per_layer_model_projection.weight": (layers * width, hidden),
        f"{root}.per_layer_projection_norm.weight": (width,),
    }
    for i in range(layers):
        head = c.global_head_dim if c.full(i) else c.head_dim
        doubled = c.use_double_wide_mlp and c.owner(i) != i
        size = {"E": hidden, "P": width, "D": head, "1": 1, "Q": c.num_attention_heads * head,
                "K": c.num_key_value_heads * head, "M": c.intermediate_size * (2 if doubled else 1)}
        for tensor, letters in _LAYER_TENSORS:
            named[f"{root}.layers.{i}.{tensor}"] = tuple(size[letter] for letter in letters)
    return named

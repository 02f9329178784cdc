"""Gemma 4's text decoder on the shared decoder (iron/applications/gemma4/model.py:42-246).

Sliding-window and global layers alternate as ``layer_types`` says; a global layer has its own
head size and a RoPE that turns only the first quarter of its pairs; q, k and v are RMS-normed per
head and attention is unscaled; every block's output is normed again before its residual
(``SandwichLayer``); the last ``num_kv_shared_layers`` layers attend over an earlier layer's cache
and may have a double-wide MLP; every layer gates in a per-layer input made of the token's own
row of a per-layer table and a projection of the embeddings (``PleLayer``); the logits are capped
by a tanh.  The vision and audio towers are not built: a multimodal checkpoint's text decoder
loads from its ``model.language_model`` tensors.
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


def _dig(data: dict, path: str):
    for key in path.split("."):
        if not isinstance(data, dict) or key not in data:
            return None
        data = data[key]
    return data


@dataclasses.dataclass(frozen=True)
class Gemma4Config(DecoderConfig):
    """``DecoderConfig`` as a checkpoint's ``text_config`` holds it, with the global layers' heads
    and RoPE, the shared caches, the per-layer inputs and the logits' cap."""

    precision: Precision = dataclasses.field(default=Precision.MEDIUM, kw_only=True)
    hidden_act: str = "gelu_pytorch_tanh"
    layer_types: tuple[str, ...] = dataclasses.field(kw_only=True)
    global_head_dim: int = dataclasses.field(default=512, kw_only=True)
    global_rope_theta: float = dataclasses.field(default=1000000.0, kw_only=True)
    partial_rotary_factor: float = dataclasses.field(default=0.25, kw_only=True)
    num_kv_shared_layers: int = dataclasses.field(default=0, kw_only=True)
    use_double_wide_mlp: bool = dataclasses.field(default=False, kw_only=True)
    ple_dim: int = dataclasses.field(default=256, kw_only=True)
    final_logit_softcapping: float | None = dataclasses.field(default=None, kw_only=True)
    # The placeholders a tower's soft tokens would replace, which the per-layer inputs read as the
    # padding token.
    pad_token_id: int = dataclasses.field(default=0, kw_only=True)
    image_token_id: int | None = dataclasses.field(default=None, kw_only=True)
    audio_token_id: int | None = dataclasses.field(default=None, kw_only=True)
    video_token_id: int | None = dataclasses.field(default=None, kw_only=True)

    # Where ``text_config`` holds a field under another name or deeper; a leading "/" is the file's
    # top level.
    PATHS = {
        "eps": "rms_norm_eps", "max_seq_len": "max_position_embeddings", "hidden_act": "hidden_activation",
        "rope_theta": "rope_parameters.sliding_attention.rope_theta",
        "global_rope_theta": "rope_parameters.full_attention.rope_theta",
        "partial_rotary_factor": "rope_parameters.full_attention.partial_rotary_factor",
        "ple_dim": "hidden_size_per_layer_input",
        "image_token_id": "/image_token_id", "audio_token_id": "/audio_token_id", "video_token_id": "/video_token_id",
    }
    NOT_JSON = ("precision", "prefill_chunk", "rope_scaling")

    @classmethod
    def from_json(cls, data: dict, source="config.json") -> "Gemma4Config":
        """The fields of a parsed ``config.json`` (iron/applications/gemma4/model.py:89-125).

        Raises:
            ValueError: the file asks for what is not built here (keys equal to values, experts, an
                attention soft-cap, bidirectional text, a per-layer vocabulary other than the
                embedding's, RoPE other than the sliding layers' default and the global ones'
                proportional), or lacks a field that has no default.
        """
        text = dict(data.get("text_config", {}))
        for key in ("attention_k_eq_v", "enable_moe_block", "attn_logit_softcapping"):
            if text.get(key):
                raise ValueError(f"{source}: {key} {text[key]!r} is not built here")
        # "vision" makes only image tokens bidirectional; text has none.
        bidirectional = text.get("use_bidirectional_attention")
        if bidirectional not in (None, False, "vision"):
            raise ValueError(f"{source}: bidirectional attention {bidirectional!r} is not built here")
        per_layer = text.get("vocab_size_per_layer_input", text.get("vocab_size"))
        if per_layer != text.get("vocab_size"):
            raise ValueError(f"{source}: vocab_size_per_layer_input {per_layer} other than vocab_size "
                             f"{text.get('vocab_size')} is not built here")
        rope = text.get("rope_parameters", {})
        for kind, built in (("sliding_attention", "default"), ("full_attention", "proportional")):
            got = rope.get(kind, {}).get("rope_type", built)
            if got != built:
                raise ValueError(f"{source}: {kind} RoPE {got!r} is not built here")
        kwargs, missing = {}, []
        for f in dataclasses.fields(cls):
            if f.name in cls.NOT_JSON:
                continue
            path = cls.PATHS.get(f.name, f.name)
            value = _dig(data, path[1:]) if path.startswith("/") else _dig(text, path)
            if value is None:
                if f.default is dataclasses.MISSING and f.default_factory is dataclasses.MISSING:
                    missing.append(path)
                continue
            kwargs[f.name] = tuple(value) if f.name == "layer_types" else value
        if missing:
            raise ValueError(f"{source} lacks {missing}")
        return cls(**kwargs)

    def to_json(self) -> dict:
        """``from_json``'s inverse: the fields under ``text_config`` (or the top level) where a
        checkpoint's ``config.json`` holds them."""
        out: dict = {"text_config": {}}
        for f in dataclasses.fields(self):
            value = getattr(self, f.name)
            if f.name in self.NOT_JSON or value is None:
                continue
            path = self.PATHS.get(f.name, f.name)
            at = out if path.startswith("/") else out["text_config"]
            *parents, leaf = path.lstrip("/").split(".")
            for key in parents:
                at = at.setdefault(key, {})
            at[leaf] = list(value) if isinstance(value, tuple) else value
        return out

    def full(self, i: int) -> bool:
        """Whether layer ``i`` is global."""
        return self.layer_types[i] == "full_attention"

    def owner(self, i: int) -> int:
        """The layer whose cache layer ``i`` attends over: its own, or for a shared layer the last
        one of its kind before the shared ones."""
        first = self.num_hidden_layers - self.num_kv_shared_layers
        if i < first:
            return i
        owners = [j for j in range(first) if self.full(j) == self.full(i)]
        if not owners:
            raise ValueError(f"Gemma4Config: shared layer {i} has no earlier layer of its kind")
        return owners[-1]


class Gemma4Decoder(Decoder):
    """``Decoder`` and the per-layer inputs' token table, projection and norm."""

    def __init__(self, c: Gemma4Config, layer):
        super().__init__(c, layer)
        L, P, E = c.num_hidden_layers, c.ple_dim, c.hidden_size
        # Dropped once the loaded table has been split into the layers'.
        self.embed_tokens_per_layer = Embedding(c.vocab_size, L * P)
        self.per_layer_model_projection = Linear(E, L * P, False, precision=c.precision)
        self.per_layer_projection_norm = RMSNorm(P, c.eps)


class Gemma4Layer(PleLayer):
    """Layer ``i``: unscaled attention over normed q, k and v -- a global layer's heads and whole
    context where it is one, else within the window -- and a double-wide MLP on a shared layer
    where ``use_double_wide_mlp``."""

    def __init__(self, c: Gemma4Config, i: int):
        heads = dataclasses.replace(c, head_dim=c.global_head_dim) if c.full(i) else c
        mlp = None
        if c.use_double_wide_mlp and c.owner(i) != i:
            mlp = GatedMLP(dataclasses.replace(c, intermediate_size=2 * c.intermediate_size))
        super().__init__(c, i, Attention(heads, i, norms="qkv"), mlp, KVCache(heads, None if c.full(i) else c.window))
        self.self_attn.scaling = 1.0


def _host_array(array) -> np.ndarray:
    """A loaded weight as a float32 array of bf16 values (a checkpoint hands over torch tensors)."""
    if type(array).__module__.startswith("torch"):
        return from_torch(array)
    return np.asarray(array, dtype=np.float32)


class _StillPairs:
    """Proportional RoPE: the pairs past ``turned`` stand still (frequency zero)."""

    def __init__(self, turned: int):
        self.turned = turned

    def __call__(self, inv_freq: np.ndarray) -> np.ndarray:
        return np.where(np.arange(inv_freq.size) < self.turned, inv_freq, 0)


class Gemma4(CausalLM):
    """Gemma 4's text decoder on ``config``'s shape and a checkpoint's ``weights`` (by tensor name;
    the decoder's are under ``model.language_model``, the towers' are left out)."""

    config_class = Gemma4Config
    decoder_class = Gemma4Decoder
    layer_class = Gemma4Layer

    def __init__(self, config: Gemma4Config, weights):
        text = {"model." + name[len(PREFIX):]: t for name, t in weights.items() if name.startswith(PREFIX)}
        if "lm_head.weight" in weights:
            text["lm_head.weight"] = weights["lm_head.weight"]
        super().__init__(config, text)
        c = config
        turned = int(c.partial_rotary_factor * c.global_head_dim // 2)
        rope = Rope(dataclasses.replace(c, head_dim=c.global_head_dim, rope_theta=c.global_rope_theta,
                                        rope_scaling=_StillPairs(turned)))
        for i, layer in enumerate(self.layers):
            if c.full(i):
                layer.rope = rope
            if c.owner(i) != i:
                attention = layer.self_attn
                attention.k_proj = attention.v_proj = attention.k_norm = None
                layer.cache = self.layers[c.owner(i)].cache

    def load_state_dict(self, tree, *, path: str = "") -> None:
        c, m = self.config, self.model
        # A shared layer's k/v projections and k norm are never read: a checkpoint that ships them
        # loads them (they are dropped once the caches are shared), one that does not need not.
        for i, layer in enumerate(m.layers):
            if c.owner(i) != i and f"{path}model.layers.{i}.self_attn.k_proj.weight" not in tree:
                layer.self_attn.k_proj = layer.self_attn.v_proj = layer.self_attn.k_norm = None
        super().load_state_dict(tree, path=path)
        P, E = c.ple_dim, c.hidden_size
        scale = round_bf16(np.float32(np.sqrt(P)))
        table = _host_array(m.embed_tokens_per_layer.weight.array)
        placeholders = [t for t in (c.image_token_id, c.audio_token_id, c.video_token_id) if t is not None]
        for i, layer in enumerate(m.layers):
            # A layer's own columns, scaled, contiguous: one gather a layer.
            rows = table[:, i * P : (i + 1) * P] * scale
            rows[placeholders] = rows[c.pad_token_id]
            layer.per_layer_embedding = iron.param(round_bf16(rows))
            # The row every row of the layer's output is multiplied by.
            scalar = _host_array(layer.layer_scalar.array)
            layer.scale = iron.param(round_bf16(np.full(E, scalar[0], np.float32)))
        m.embed_tokens_per_layer = None

    def lookup(self, ids):
        # The embedding times sqrt(hidden_size), a constant row in the weights' dtype.
        return super().lookup(ids) * float(np.sqrt(self.config.hidden_size))

    def layer(self, call, i, w, x):
        """Layer ``i`` on ``x``, its per-layer input made from the call's embeddings and ids."""
        c, m, P = self.config, self.model, self.config.ple_dim
        projection = m.per_layer_model_projection.weight[i * P : (i + 1) * P]
        ple = F.linear(call.embeddings, projection, precision=c.precision)
        rows = call.embeddings.elements // c.hidden_size
        # The projection's hidden_size ** -0.5 folded into the norm's epsilon:
        # RMSNorm(s * y, eps) is RMSNorm(y, eps / s ** 2).
        ple = F.rms_norm(ple.reshape(rows, P), (P,), m.per_layer_projection_norm.weight, c.eps * c.hidden_size)
        token = Copy.step(iron.weight(w.per_layer_embedding)[call.ids])
        return w(x, call, (ple + token.reshape(ple.shape)) * 2**-0.5)

    def head(self, x):
        """The tied head's logits, capped by a tanh where the config says."""
        logits, cap = super().head(x), self.config.final_logit_softcapping
        return logits if cap is None else Tanh.step(logits * (1 / cap)) * cap


def shapes(config: Gemma4Config) -> dict[str, tuple[int, ...]]:
    """Each tensor of a Hugging Face Gemma 4 checkpoint's text decoder of ``config``'s shape, by
    name, in the order the reference's toy draws them
    (tests/applications/gemma4/reference/test.py:60-108)."""
    c = config
    L, E, P, V = c.num_hidden_layers, c.hidden_size, c.ple_dim, c.vocab_size
    H, G = c.num_attention_heads, c.num_key_value_heads
    model = PREFIX[:-1]
    out = {
        f"{model}.embed_tokens.weight": (V, E),
        f"{model}.norm.weight": (E,),
        f"{model}.embed_tokens_per_layer.weight": (V, L * P),
        f"{model}.per_layer_model_projection.weight": (L * P, E),
        f"{model}.per_layer_projection_norm.weight": (P,),
    }
    for i in range(L):
        D = c.global_head_dim if c.full(i) else c.head_dim
        M = c.intermediate_size * (2 if c.use_double_wide_mlp and c.owner(i) != i else 1)
        layer = f"{model}.layers.{i}"
        out |= {
            f"{layer}.self_attn.q_proj.weight": (H * D, E),
            f"{layer}.self_attn.o_proj.weight": (E, H * D),
            f"{layer}.self_attn.q_norm.weight": (D,),
            f"{layer}.mlp.gate_proj.weight": (M, E),
            f"{layer}.mlp.up_proj.weight": (M, E),
            f"{layer}.mlp.down_proj.weight": (E, M),
            f"{layer}.per_layer_input_gate.weight": (P, E),
            f"{layer}.per_layer_projection.weight": (E, P),
            f"{layer}.layer_scalar": (1,),
            # A shared layer's too: the checkpoint ships them, the layer never reads them.
            f"{layer}.self_attn.k_proj.weight": (G * D, E),
            f"{layer}.self_attn.v_proj.weight": (G * D, E),
            f"{layer}.self_attn.k_norm.weight": (D,),
        }
        out |= {f"{layer}.{norm}.weight": (E,) for norm in (
            "input_layernorm", "post_attention_layernorm", "pre_feedforward_layernorm",
            "post_feedforward_layernorm", "post_per_layer_input_norm")}
    return out

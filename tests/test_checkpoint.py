"""Checkpoints, configs and tokenizers read from a model's own files (iron/lm/checkpoint.py,
iron/lm/config.py:97-147, iron/lm/model.py:125-235,321-407): bit-exact against the safetensors
and torch libraries as independent writers/readers, refusals for malformed files and for pickles
that name code, and the toy Llama loaded from a directory against the reference's golden logits."""

import dataclasses
import json
import pickle
import struct

import numpy as np
import pytest

import oracle
from iron_amd.applications.llama import LLAMA_3_2_1B, Llama, LlamaConfig
from iron_amd.bf16 import round_bf16, to_bits
from iron_amd.lm.causal import OnHost
from iron_amd.lm.checkpoint import Checkpoint, leaves, nest, weights_file, write_safetensors
from tests.llama_support import SCALED, Golden, assert_close, weights

oracle.install()
torch = pytest.importorskip("torch")


def some_tensors(rng):
    return {
        "model.embed.weight": round_bf16(rng.standard_normal((7, 16), dtype=np.float32)),
        "model.layers.0.w": round_bf16(rng.standard_normal((4, 8), dtype=np.float32)),
        "model.layers.1.w": rng.standard_normal((3, 5), dtype=np.float32) + np.float32(1e-3),  # not bf16-valued: F32
        "model.half": rng.standard_normal(9).astype(np.float16),
        "model.count": np.arange(3, dtype=np.int64),
    }


def test_written_file_is_what_the_safetensors_library_reads(tmp_path):
    st = pytest.importorskip("safetensors.torch")
    t = some_tensors(np.random.default_rng(0))
    path = write_safetensors(tmp_path / "model.safetensors", t)
    theirs = st.load_file(str(path))
    assert set(theirs) == set(t)
    assert theirs["model.embed.weight"].dtype == torch.bfloat16 and theirs["model.layers.1.w"].dtype == torch.float32
    for n, a in t.items():
        assert np.array_equal(theirs[n].to(torch.float64).numpy(), a.astype(np.float64)), n
    ours = Checkpoint(path)
    assert list(ours.tensors) == list(t)
    for n, a in t.items():
        assert np.array_equal(ours.tensors[n], a) and ours.tensors[n].dtype == a.dtype, n
    assert ours.torch("model.embed.weight").dtype == torch.bfloat16
    assert np.array_equal(ours.torch("model.embed.weight").view(torch.int16).numpy().view(np.uint16),
                          to_bits(t["model.embed.weight"]))


def test_a_file_the_safetensors_library_wrote_reads_bit_for_bit(tmp_path):
    st = pytest.importorskip("safetensors.torch")
    g = torch.Generator().manual_seed(3)
    theirs = {"a.b": torch.randn(5, 6, generator=g).to(torch.bfloat16), "a.c": torch.randn(4, generator=g),
              "d": torch.randn(2, 3, generator=g).to(torch.float16)}
    st.save_file(theirs, str(tmp_path / "x.safetensors"), metadata={"format": "pt"})
    ours = Checkpoint(tmp_path / "x.safetensors")
    for n, t in theirs.items():
        assert np.array_equal(ours.tensors[n].astype(np.float64), t.to(torch.float64).numpy()), n
    assert ours.shapes()["a.b"][0] == (5, 6)


def test_a_sharded_checkpoint_merges_its_shards_and_checks_the_index(tmp_path):
    t = some_tensors(np.random.default_rng(1))
    names = list(t)
    write_safetensors(tmp_path / "model-00001-of-00002.safetensors", {n: t[n] for n in names[:2]})
    write_safetensors(tmp_path / "model-00002-of-00002.safetensors", {n: t[n] for n in names[2:]})
    index = {"weight_map": {n: f"model-0000{1 if i < 2 else 2}-of-00002.safetensors" for i, n in enumerate(names)}}
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps(index))
    assert weights_file(tmp_path).name == "model.safetensors.index.json"
    ck = Checkpoint(weights_file(tmp_path))
    assert set(ck.tensors) == set(t) and all(np.array_equal(ck.tensors[n], t[n]) for n in t)
    index["weight_map"][names[0]] = "model-00002-of-00002.safetensors"
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps(index))
    with pytest.raises(ValueError, match="the index does not name"):
        Checkpoint(tmp_path / "model.safetensors.index.json")
    index["weight_map"][names[0]] = "../elsewhere.safetensors"
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps(index))
    with pytest.raises(ValueError, match="not a file beside the index"):
        Checkpoint(tmp_path / "model.safetensors.index.json")


@pytest.mark.parametrize("header,match", [
    ({"x": {"dtype": "F8", "shape": [2], "data_offsets": [0, 2]}}, "x is F8"),
    ({"x": {"dtype": "F32", "shape": [2]}}, "no data_offsets"),
    ({"x": {"dtype": "F32", "shape": [2], "data_offsets": [0, 4]}}, "spans bytes"),
    ({"x": {"dtype": "F32", "shape": [2], "data_offsets": [0, 64]}}, "spans bytes"),
])
def test_a_malformed_header_is_refused(tmp_path, header, match):
    blob = json.dumps(header).encode()
    (tmp_path / "bad.safetensors").write_bytes(struct.pack("<Q", len(blob)) + blob + bytes(8))
    with pytest.raises(ValueError, match=match):
        Checkpoint(tmp_path / "bad.safetensors")


def test_a_pytorch_checkpoint_reads_as_data_and_runs_no_code(tmp_path):
    g = torch.Generator().manual_seed(5)
    base = torch.randn(6, 8, generator=g).to(torch.bfloat16)
    state = {"w": base, "wt": base.t(), "v": torch.randn(5, generator=g), "n": torch.tensor([3, 4]),
             "nested": {"h": torch.randn(2, 2, generator=g).to(torch.float16)}}
    torch.save(state, tmp_path / "model.pth")
    ck = Checkpoint(tmp_path / "model.pth")
    assert set(ck.tensors) == {"w", "wt", "v", "n", "nested.h"}
    assert np.array_equal(ck.tensors["w"].astype(np.float64), base.to(torch.float64).numpy())
    assert np.array_equal(ck.tensors["wt"].astype(np.float64), base.t().to(torch.float64).numpy())  # a strided view
    assert np.array_equal(ck.tensors["n"], np.array([3, 4]))
    assert np.array_equal(ck.tensors["nested.h"], state["nested"]["h"].numpy())

    # A pickle that names anything but a state dict's own globals is refused before it can run.
    import io
    import zipfile

    class Evil:
        def __reduce__(self):
            return (print, ("this must not run",))

    with zipfile.ZipFile(tmp_path / "evil.pth", "w", zipfile.ZIP_STORED) as z:
        z.writestr("archive/data.pkl", pickle.dumps({"w": Evil()}))
        z.writestr("archive/version", "3")
    with pytest.raises(pickle.UnpicklingError, match="may not load builtins.print"):
        Checkpoint(tmp_path / "evil.pth")


def test_nest_and_leaves_are_inverses_and_name_what_is_missing(tmp_path):
    flat = {"model.layers.0.w": 1, "model.layers.2.w": 2, "model.norm.weight": 3, "lm_head.weight": 4}
    tree = nest(flat, file="toy.safetensors")
    assert tree.model.layers[2].w == 2 and len(tree.model.layers) == 3 and vars(tree.model.layers[1]) == {}
    assert dict(leaves(tree)) == flat
    with pytest.raises(AttributeError, match=r"model\.embed is not in toy\.safetensors \(it has layers, norm\)"):
        tree.model.embed
    with pytest.raises(IndexError, match=r"model\.layers\.5 is not in toy\.safetensors \(it has 3\)"):
        tree.model.layers[5]
    with pytest.raises(ValueError, match="past its 1 layers"):
        nest({"layers.99.w": 0})


LLAMA_3_2_1B_JSON = {
    "architectures": ["LlamaForCausalLM"], "attention_bias": False, "attention_dropout": 0.0, "bos_token_id": 128000,
    "eos_token_id": 128001, "head_dim": 64, "hidden_act": "silu", "hidden_size": 2048, "initializer_range": 0.02,
    "intermediate_size": 8192, "max_position_embeddings": 131072, "mlp_bias": False, "model_type": "llama",
    "num_attention_heads": 32, "num_hidden_layers": 16, "num_key_value_heads": 8, "pretraining_tp": 1,
    "rms_norm_eps": 1e-05,
    "rope_scaling": {"factor": 32.0, "high_freq_factor": 4.0, "low_freq_factor": 1.0,
                     "original_max_position_embeddings": 8192, "rope_type": "llama3"},
    "rope_theta": 500000.0, "tie_word_embeddings": True, "torch_dtype": "bfloat16", "use_cache": True,
    "vocab_size": 128256,
}


def test_a_config_is_read_from_the_checkpoint_s_config_json(tmp_path):
    (tmp_path / "config.json").write_text(json.dumps(LLAMA_3_2_1B_JSON))
    for where in (tmp_path, tmp_path / "config.json", tmp_path / "model.safetensors"):
        assert LlamaConfig.from_checkpoint(where) == LLAMA_3_2_1B
    again = LlamaConfig.from_json(LLAMA_3_2_1B.to_json())
    assert again == LLAMA_3_2_1B
    lacking = {k: v for k, v in LLAMA_3_2_1B_JSON.items() if k not in ("vocab_size", "rope_theta")}
    with pytest.raises(ValueError, match=r"lacks \['vocab_size', 'rope_theta'\]"):
        LlamaConfig.from_json(lacking, "there/config.json")
    with pytest.raises(ValueError, match="no RoPE table here builds it"):
        LlamaConfig.from_json({**LLAMA_3_2_1B_JSON, "rope_scaling": {"rope_type": "yarn", "factor": 2.0}})
    wide = LlamaConfig.from_json({**LLAMA_3_2_1B_JSON, "hidden_size": 3072})
    assert wide.precision.name == "HIGH" and LLAMA_3_2_1B.precision.name == "MEDIUM"
    with pytest.raises(FileNotFoundError):
        LlamaConfig.from_checkpoint(tmp_path / "nowhere" / "model.safetensors")


class HostLlama(OnHost, Llama):
    pass


def toy_directory(tmp_path, with_tokenizer=True):
    config = SCALED
    (tmp_path / "config.json").write_text(json.dumps({**config.to_json(), "eos_token_id": [1000, 1001]}))
    write_safetensors(tmp_path / "model.safetensors", weights(config))
    if with_tokenizer:
        tokenizers = pytest.importorskip("tokenizers")
        from tokenizers import models, pre_tokenizers, processors

        vocab = {f"w{i}": i for i in range(config.vocab_size - 1)} | {"<s>": config.vocab_size - 1}
        tok = tokenizers.Tokenizer(models.WordLevel(vocab, unk_token="w0"))
        tok.pre_tokenizer = pre_tokenizers.Whitespace()
        tok.add_special_tokens(["<s>"])  # so a rendered chat's "<s>" is its own id, as a checkpoint's is
        tok.post_processor = processors.TemplateProcessing(single="<s> $A", special_tokens=[("<s>", config.vocab_size - 1)])
        tok.save(str(tmp_path / "tokenizer.json"))
        (tmp_path / "tokenizer_config.json").write_text(json.dumps({
            "bos_token": "<s>",
            "chat_template": "{{ bos_token }}{% for m in messages %}{{ m['content'] }} {% endfor %}w7"}))
    return tmp_path


def test_the_toy_loads_from_its_directory_and_matches_the_golden(tmp_path):
    directory = toy_directory(tmp_path)
    model = HostLlama.from_checkpoint(directory)
    assert model.config == SCALED and model.eos == {1000, 1001}
    model.load_versions()
    prompt = np.random.default_rng(7).integers(0, SCALED.vocab_size, 8)
    assert_close(model.logits(prompt), Golden().logits(prompt))
    shorter = HostLlama.from_checkpoint(directory, max_seq_len=128, prefill_chunk=64)
    assert shorter.config.max_seq_len == 128 and shorter.config.prefill_chunk == 64
    with pytest.raises(ValueError, match="past the model's 256"):
        HostLlama.from_checkpoint(directory, max_seq_len=512)
    # A tensor the model does not hold, or one it lacks, is named.
    w = weights(SCALED)
    write_safetensors(tmp_path / "model.safetensors", {**w, "model.extra.weight": np.zeros(4, np.float32)})
    with pytest.raises(ValueError, match="extra model.extra.weight"):
        HostLlama.from_checkpoint(directory)
    w.pop("model.norm.weight")
    write_safetensors(tmp_path / "model.safetensors", w)
    with pytest.raises(ValueError, match="missing model.norm.weight"):
        HostLlama.from_checkpoint(directory)


def test_text_in_text_out_through_the_checkpoint_s_tokenizer(tmp_path):
    model = HostLlama.from_checkpoint(toy_directory(tmp_path))
    model.load_versions()
    tk = model.tokenizer
    assert tk("w5 w9") == [SCALED.vocab_size - 1, 5, 9] and tk.decode([5, 9]) == "w5 w9"
    assert tk.chat([{"role": "user", "content": "w3 w4"}]) == [SCALED.vocab_size - 1, 3, 4, 7]
    ids = model.generate(tk("w5 w9"), 4)
    text = model.generate("w5 w9", 4)
    assert text == tk.decode([t for t in ids if t not in model.eos])
    assert isinstance(model.generate([{"role": "user", "content": "w3 w4"}], 2), str)
    bare = HostLlama(SCALED, weights())
    bare.load_versions()
    with pytest.raises(ValueError, match="takes the checkpoint's tokenizer"):
        bare.generate("w5", 2)

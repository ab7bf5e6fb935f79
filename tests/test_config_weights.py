"""Configuration, registry and weight loading (no GPU)."""

import json

import pytest
import torch

import bitwise_amd as bw
from bitwise_amd import registry
from bitwise_amd.config.llama import ConfigError, LlamaConfig
from bitwise_amd.model import model_spec
from bitwise_amd.weights import loader, safetensors_io
from tiny import TINY_A, TINY_B


def test_keys_and_defaults_follow_the_converter():
    """tools/convert.py:55-80: kv heads default to heads, head_dim to hidden/heads, theta 10000,
    eps 1e-6, untied, a list of eos ids means the first."""
    c = LlamaConfig.from_dict({"architectures": ["LlamaForCausalLM"], "vocab_size": 100, "hidden_size": 96,
                               "num_hidden_layers": 2, "num_attention_heads": 3, "intermediate_size": 224,
                               "eos_token_id": [7, 9]})
    assert (c.num_key_value_heads, c.head_dim, c.rope_theta, c.rms_norm_eps) == (3, 32, 10000.0, 1e-6)
    assert c.tie_word_embeddings is False and c.eos_token_id == 7 and c.bos_token_id == -1
    assert (c.q_dim, c.kv_dim) == (96, 96)
    b = LlamaConfig.from_dict(TINY_B)
    assert (b.num_key_value_heads, b.head_dim, b.q_dim, b.kv_dim, b.rms_norm_eps) == (1, 32, 96, 32, 1e-6)
    assert LlamaConfig.from_dict(b.to_dict()) == b


@pytest.mark.parametrize("patch, match", [
    ({"rope_scaling": {"type": "linear", "factor": 2}}, "rope_scaling"),
    ({"attention_bias": True}, "attention_bias"),
    ({"hidden_act": "gelu"}, "hidden_act"),
    ({"num_key_value_heads": 3}, "multiple"),
    ({"head_dim": 15}, "even"),
    ({"vocab_size": "many"}, "integer"),
])
def test_what_the_engine_cannot_run_is_refused(patch, match):
    with pytest.raises(ConfigError, match=match):
        LlamaConfig.from_dict(dict(TINY_A, **patch))


def test_missing_key_and_unknown_architecture():
    d = dict(TINY_A)
    del d["intermediate_size"]
    with pytest.raises(ConfigError, match="intermediate_size"):
        LlamaConfig.from_dict(d)
    with pytest.raises(ConfigError, match="unsupported architecture Qwen2ForCausalLM"):
        registry.architecture_of(dict(TINY_A, architectures=["Qwen2ForCausalLM"]))
    assert registry.architecture_of(TINY_A).name == "LlamaForCausalLM"


def test_tensor_names_are_the_checkpoints_own():
    """src/model.cpp:136-171; the head has a tensor of its own only when untied."""
    a, b = bw.describe(TINY_A), bw.describe(TINY_B)
    assert "lm_head.weight" not in a and b["lm_head.weight"].shape == (500, 96)
    assert a["model.layers.1.self_attn.k_proj.weight"].shape == (32, 64)
    assert b["model.layers.2.mlp.down_proj.weight"].shape == (96, 224)
    assert b["model.layers.0.self_attn.q_proj.weight"].shape == (96, 96)
    assert a["model.norm.weight"].kind == "norm" and a["model.embed_tokens.weight"].shape == (256, 64)
    assert len(a) == 1 + 9 * 2 + 1 and len(b) == 1 + 9 * 3 + 2


def test_random_folder_roundtrip_and_distribution(tmp_path):
    folder = bw.write_random_model(tmp_path / "m", TINY_B, seed=1, sigma=0.05)
    assert json.loads((folder / "config.json").read_text())["num_key_value_heads"] == 1
    specs = bw.describe(TINY_B)
    w = loader.load_folder(folder, specs)
    assert set(w) == set(specs) and all(t.dtype == torch.bfloat16 for t in w.values())
    big = w["model.embed_tokens.weight"].float()
    assert abs(big.std().item() - 0.05) < 0.005 and abs(big.mean().item()) < 0.002
    norm = w["model.layers.0.input_layernorm.weight"].float()
    assert abs(norm.mean().item() - 1.0) < 0.05 and 0.05 < norm.std().item() < 0.15
    again = dict(loader.random_tensors(specs, 1, 0.05))
    assert all(torch.equal(again[k], w[k]) for k in w)           # same seed, same bits
    other = dict(loader.random_tensors(specs, 2, 0.05))
    assert not torch.equal(other["model.norm.weight"], w["model.norm.weight"])
    from safetensors.torch import load_file                       # the file is a regular safetensors file
    lib = load_file(str(folder / "model.safetensors"))
    assert all(torch.equal(lib[k], w[k]) for k in w)


def test_stored_dtypes_are_kept(tmp_path):
    specs = bw.describe(TINY_A)
    tensors = dict(loader.random_tensors(specs, 0))
    tensors["model.norm.weight"] = tensors["model.norm.weight"].float()                   # 32-bit stays 32-bit
    tensors["model.layers.0.mlp.up_proj.weight"] = tensors["model.layers.0.mlp.up_proj.weight"].half()
    safetensors_io.write_file(tmp_path / "model.safetensors", tensors.items())
    w = loader.load_folder(tmp_path, specs)
    assert w["model.norm.weight"].dtype == torch.float32
    assert w["model.layers.0.mlp.up_proj.weight"].dtype == torch.float32                  # float16 is widened
    assert w["model.embed_tokens.weight"].dtype == torch.bfloat16


def test_one_error_lists_missing_unexpected_and_misshapen(tmp_path):
    specs = bw.describe(TINY_A)
    tensors = dict(loader.random_tensors(specs, 0))
    del tensors["model.layers.1.mlp.down_proj.weight"]
    del tensors["model.norm.weight"]
    tensors["model.layers.0.self_attn.bias"] = torch.zeros(64, dtype=torch.bfloat16)     # nothing reads it
    tensors["model.layers.0.self_attn.q_proj.weight"] = torch.zeros(64, 32, dtype=torch.bfloat16)
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)             # exporter's buffer: ignored
    safetensors_io.write_file(tmp_path / "model.safetensors", tensors.items())
    spec = model_spec(TINY_A)
    with pytest.raises(bw.WeightError) as e:
        loader.load_folder(tmp_path, specs, spec.ignored_tensor_suffixes, spec.unused_tensors)
    msg = str(e.value)
    assert "missing tensors (2)" in msg and "model.norm.weight" in msg and "model.layers.1.mlp.down_proj.weight" in msg
    assert "unexpected tensors (1): model.layers.0.self_attn.bias" in msg and "inv_freq" not in msg
    assert "model.layers.0.self_attn.q_proj.weight: stored (64, 32), the configuration needs (64, 64)" in msg


def test_a_tied_checkpoint_that_stores_the_head_loads_with_a_warning(tmp_path):
    """The reference reads lm_head.weight only when the head is not tied (src/model.cpp:170-171); a tied
    checkpoint that stores it anyway is used without it, and says so.  An untied model still needs it, and a
    tensor that no configuration of the architecture reads is still an error."""
    specs, spec = bw.describe(TINY_A), model_spec(TINY_A)
    assert spec.unused_tensors == ("lm_head.weight",) and model_spec(TINY_B).unused_tensors == ()
    tensors = dict(loader.random_tensors(specs, 0))
    tensors["lm_head.weight"] = torch.zeros(256, 64, dtype=torch.bfloat16)
    safetensors_io.write_file(tmp_path / "model.safetensors", tensors.items())
    with pytest.warns(loader.UnusedTensorWarning, match="lm_head.weight"):
        w = loader.load_folder(tmp_path, specs, spec.ignored_tensor_suffixes, spec.unused_tensors)
    assert set(w) == set(specs)
    with pytest.raises(bw.WeightError, match="unexpected tensors \\(1\\): lm_head.weight"):
        loader.load_folder(tmp_path, specs)                      # an architecture that does not know the name


def test_broken_files(tmp_path):
    with pytest.raises(safetensors_io.SafetensorsError, match="no \\*.safetensors"):
        loader.load_folder(tmp_path, {})
    (tmp_path / "model.safetensors").write_bytes(b"\x10\x00\x00")
    with pytest.raises(safetensors_io.SafetensorsError, match="too short"):
        loader.load_folder(tmp_path, {})
    specs = bw.describe(TINY_A)
    safetensors_io.write_file(tmp_path / "model.safetensors", loader.random_tensors(specs, 0))
    raw = (tmp_path / "model.safetensors").read_bytes()
    (tmp_path / "model.safetensors").write_bytes(raw[:-100])
    with pytest.raises(safetensors_io.SafetensorsError, match="truncated tensor"):
        loader.load_folder(tmp_path, specs)
    # offsets that run backwards, or two tensors on the same bytes
    import json
    import struct

    def write(header):
        text = json.dumps(header).encode()
        (tmp_path / "model.safetensors").write_bytes(struct.pack("<Q", len(text)) + text + bytes(64))

    write({"a": {"dtype": "F32", "shape": [4], "data_offsets": [16, 0]}})
    with pytest.raises(safetensors_io.SafetensorsError, match="run backwards"):
        safetensors_io.read_file(tmp_path / "model.safetensors")
    write({"a": {"dtype": "F32", "shape": [4], "data_offsets": [0, 16]}, "b": {"dtype": "F32", "shape": [4], "data_offsets": [8, 24]}})
    with pytest.raises(safetensors_io.SafetensorsError, match="overlap"):
        safetensors_io.read_file(tmp_path / "model.safetensors")
    with pytest.raises(ConfigError, match="cannot open"):
        registry.read_config(tmp_path / "nowhere")

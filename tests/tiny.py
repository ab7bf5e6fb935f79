"""Two tiny Llama configurations that differ in every size and option, and helpers that make
model folders for them in temporary directories."""

from __future__ import annotations

import json
from pathlib import Path
from typing import Dict

import torch

# layers, width, heads / kv heads (group 2), head size, feed-forward, vocabulary, rotary base,
# eps, tied head, positions
TINY_A = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama", "hidden_act": "silu",
    "vocab_size": 256, "hidden_size": 64, "num_hidden_layers": 2, "num_attention_heads": 4,
    "num_key_value_heads": 2, "head_dim": 16, "intermediate_size": 128, "rope_theta": 10000.0,
    "rms_norm_eps": 1e-5, "tie_word_embeddings": True, "max_position_embeddings": 128,
    "bos_token_id": 1, "eos_token_id": 2,
}
# three layers, width 96 (no power of two), 3 heads on 1 kv head (group 3), head size 32,
# feed-forward 224, vocabulary 500 (no multiple of 16), other base and eps, untied head
TINY_B = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama", "hidden_act": "silu",
    "vocab_size": 500, "hidden_size": 96, "num_hidden_layers": 3, "num_attention_heads": 3,
    "num_key_value_heads": 1, "head_dim": 32, "intermediate_size": 224, "rope_theta": 100000.0,
    "rms_norm_eps": 1e-6, "tie_word_embeddings": False, "max_position_embeddings": 256,
    "bos_token_id": 0, "eos_token_id": 3,
}
# a longer-context variant of A's shape with head size 64 and 8 heads on 2 kv heads, for tests that
# need hundreds of keys
TINY_LONG = dict(TINY_A, hidden_size=128, num_attention_heads=8, num_key_value_heads=2, head_dim=64,
                 intermediate_size=96, vocab_size=320, max_position_embeddings=1024, num_hidden_layers=2,
                 tie_word_embeddings=False)

CONFIGS = {"A": (TINY_A, 0, 0.02, 16), "B": (TINY_B, 1, 0.05, 8), "LONG": (TINY_LONG, 2, 0.05, 16)}


def make_folder(tmp: Path, name: str, weight_dtype: str = "bfloat16") -> Path:
    """Write config.json and model.safetensors of a tiny configuration with its own seed and
    weight scale; returns the folder."""
    from bitwise_amd.model import write_random_model

    cfg, seed, sigma, _ = CONFIGS[name]
    folder = Path(tmp) / f"tiny_{name}_{weight_dtype}"
    if not (folder / "model.safetensors").exists():
        write_random_model(folder, cfg, seed, sigma, weight_dtype)
    return folder


def read_weights(folder: Path) -> Dict[str, torch.Tensor]:
    """The folder's tensors through the safetensors package (not the engine's reader)."""
    from safetensors.torch import load_file

    return load_file(str(Path(folder) / "model.safetensors"))


def read_config(folder: Path) -> dict:
    return json.loads((Path(folder) / "config.json").read_text())


def plain_mode(dtype: str) -> dict:
    """Keyword arguments that make the plain float64 model the counterpart of a precision mode: in bfloat16
    mode activations are rounded to bfloat16 where the engine stores them so, and attention weights are rounded
    within partitions of 64 keys at absolute positions (the engine's definition of that mode); the 32-bit mode
    rounds nothing."""
    import plain_llama as pl

    return {"rnd": pl.round_bf16, "partition": 64} if dtype == "bfloat16" else {"rnd": pl.identity}

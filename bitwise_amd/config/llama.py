"""Typed configuration of the Llama decoder, read from the keys of its own config.json.

Keys and defaults follow the reference's converter (tools/convert.py:55-80): the
architecture name is ``architectures[0]``, ``num_key_value_heads`` defaults to the
number of heads, ``head_dim`` to ``hidden_size // num_attention_heads``,
``rope_theta`` to 10000.0, ``rms_norm_eps`` to 1e-6, ``tie_word_embeddings`` to
False, a list ``eos_token_id`` means its first element, and a truthy
``rope_scaling`` is refused (tools/convert.py:59-60).  ``max_position_embeddings``
is not read by the reference; here it bounds the rotary table and request lengths.
"""

from __future__ import annotations

import json
from dataclasses import dataclass, fields
from pathlib import Path
from typing import Any, Dict, Mapping


class ConfigError(ValueError):
    """A config.json that this engine cannot run, with the offending key named."""


def _require_int(d: Mapping[str, Any], key: str, minimum: int = 1) -> int:
    if key not in d:
        raise ConfigError(f"config.json lacks required key '{key}'")
    v = d[key]
    if isinstance(v, bool) or not isinstance(v, int):
        raise ConfigError(f"config.json key '{key}' must be an integer, got {v!r}")
    if v < minimum:
        raise ConfigError(f"config.json key '{key}' must be >= {minimum}, got {v}")
    return v


@dataclass(frozen=True)
class LlamaConfig:
    architecture: str
    vocab_size: int
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    rope_theta: float
    rms_norm_eps: float
    tie_word_embeddings: bool
    max_position_embeddings: int
    bos_token_id: int
    eos_token_id: int

    # ---- derived sizes (reference: ModelConfig::q_dim / kv_dim, src/model.h:29-30)
    @property
    def q_dim(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_dim(self) -> int:
        return self.num_key_value_heads * self.head_dim

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "LlamaConfig":
        archs = d.get("architectures")
        if not isinstance(archs, (list, tuple)) or not archs or not isinstance(archs[0], str):
            raise ConfigError("config.json lacks 'architectures': [name]")
        heads = _require_int(d, "num_attention_heads")
        hidden = _require_int(d, "hidden_size")
        kv_heads = d.get("num_key_value_heads")
        if kv_heads is None:
            kv_heads = heads
        head_dim = d.get("head_dim")
        if not head_dim:
            if hidden % heads:
                raise ConfigError(
                    f"hidden_size {hidden} is not divisible by num_attention_heads {heads} and no head_dim is given")
            head_dim = hidden // heads
        if d.get("rope_scaling"):
            raise ConfigError("rope_scaling is not supported (the reference refuses it as well)")
        for key in ("attention_bias", "mlp_bias"):
            if d.get(key):
                raise ConfigError(f"{key}=true is not supported by the Llama parts of this engine")
        act = d.get("hidden_act", "silu")
        if act != "silu":
            raise ConfigError(f"hidden_act '{act}' is not supported; the feed-forward is SwiGLU with SiLU")
        eos = d.get("eos_token_id", -1)
        if isinstance(eos, (list, tuple)):
            eos = eos[0] if eos else -1
        bos = d.get("bos_token_id", -1)
        cfg = cls(
            architecture=archs[0],
            vocab_size=_require_int(d, "vocab_size"),
            hidden_size=hidden,
            num_hidden_layers=_require_int(d, "num_hidden_layers"),
            num_attention_heads=heads,
            num_key_value_heads=int(kv_heads),
            head_dim=int(head_dim),
            intermediate_size=_require_int(d, "intermediate_size"),
            rope_theta=float(d.get("rope_theta", 10000.0)),
            rms_norm_eps=float(d.get("rms_norm_eps", 1e-6)),
            tie_word_embeddings=bool(d.get("tie_word_embeddings", False)),
            max_position_embeddings=int(d.get("max_position_embeddings", 2048)),
            bos_token_id=-1 if bos is None else int(bos),
            eos_token_id=-1 if eos is None else int(eos),
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.num_key_value_heads < 1 or self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"num_attention_heads {self.num_attention_heads} is not a multiple of "
                f"num_key_value_heads {self.num_key_value_heads}")
        if self.head_dim < 2 or self.head_dim % 2:
            raise ConfigError(f"head_dim {self.head_dim} must be even (rotary pairs i, i + head_dim/2)")
        if self.rope_theta <= 0:
            raise ConfigError(f"rope_theta must be positive, got {self.rope_theta}")
        if self.rms_norm_eps < 0:
            raise ConfigError(f"rms_norm_eps must not be negative, got {self.rms_norm_eps}")
        if self.max_position_embeddings < 1:
            raise ConfigError("max_position_embeddings must be >= 1")

    def to_dict(self) -> Dict[str, Any]:
        """The config.json form (the same keys that from_dict reads)."""
        out: Dict[str, Any] = {"architectures": [self.architecture], "model_type": "llama", "hidden_act": "silu"}
        for f in fields(self):
            if f.name != "architecture":
                out[f.name] = getattr(self, f.name)
        return out

    @classmethod
    def from_json_file(cls, path: str | Path) -> "LlamaConfig":
        return cls.from_dict(json.loads(Path(path).read_text()))

"""The Llama decoder (SmolLM2 family) as a ModelSpec: pre-norm blocks of grouped-query
attention with rotary encoding and a SwiGLU feed-forward, final RMSNorm, a head that may
be tied to the embedding (src/model.cpp:267-322, :170).  Tensor names are the checkpoint's
(src/model.cpp:136-171)."""

from __future__ import annotations

from ..config.llama import LlamaConfig
from ..parts.base import LayerCall, LayerSpec, ModelSpec, PartSpec


# The sizes of the reference simulator's tiny model (sim/simulate.cpp:64-79) as a Llama (no biases): small enough
# that a solo run of every request of a randomized scenario takes milliseconds, a vocabulary small enough that
# an end-of-sequence token is drawn now and then.
TINY_LLAMA = {
    "architectures": ["LlamaForCausalLM"], "vocab_size": 97, "hidden_size": 64, "num_hidden_layers": 2,
    "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 16, "intermediate_size": 512,
    "rope_theta": 10000.0, "rms_norm_eps": 1e-6, "tie_word_embeddings": False, "max_position_embeddings": 256,
    "eos_token_id": 3,
}


def llama_spec(cfg: LlamaConfig) -> ModelSpec:
    position = PartSpec("rope", {"theta": cfg.rope_theta, "head_dim": cfg.head_dim,
                                 "max_positions": cfg.max_position_embeddings})
    layers = []
    for i in range(cfg.num_hidden_layers):
        pre = f"model.layers.{i}."
        layers.append(LayerSpec.prenorm(
            mixer=PartSpec("attention", {"width": cfg.hidden_size, "heads": cfg.num_attention_heads,
                                         "kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
                                         "window": None, "position": position}, pre + "self_attn."),
            feed_forward=PartSpec("swiglu", {"width": cfg.hidden_size, "inter": cfg.intermediate_size}, pre + "mlp."),
            mixer_norm=PartSpec("rmsnorm", {"width": cfg.hidden_size, "eps": cfg.rms_norm_eps},
                                pre + "input_layernorm."),
            ffn_norm=PartSpec("rmsnorm", {"width": cfg.hidden_size, "eps": cfg.rms_norm_eps},
                              pre + "post_attention_layernorm."),
        ))
    return ModelSpec(
        architecture=cfg.architecture,
        vocab_size=cfg.vocab_size,
        width=cfg.hidden_size,
        embedding=PartSpec("embedding", {"vocab": cfg.vocab_size, "width": cfg.hidden_size}, "model.embed_tokens."),
        layers=layers,
        schedule=[LayerCall(layer=i, cache=i) for i in range(cfg.num_hidden_layers)],
        final_norm=PartSpec("rmsnorm", {"width": cfg.hidden_size, "eps": cfg.rms_norm_eps}, "model.norm."),
        lm_head=PartSpec("lm_head", {"vocab": cfg.vocab_size, "width": cfg.hidden_size,
                                     "tied": cfg.tie_word_embeddings}, "lm_head."),
        max_positions=cfg.max_position_embeddings,
        bos_token_id=cfg.bos_token_id,
        eos_token_id=cfg.eos_token_id,
        # exporters store the rotary frequencies as a buffer; a tied checkpoint may still carry the
        # head's matrix, which the reference never reads then (src/model.cpp:170-171)
        ignored_tensor_suffixes=("rotary_emb.inv_freq",),
        unused_tensors=("lm_head.weight",) if cfg.tie_word_embeddings else (),
    )

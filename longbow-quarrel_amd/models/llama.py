"""The Llama 3 dense decoder as a `ModelSpec`: every layer a pre-norm block of
grouped-query attention with rotary positions and a SwiGLU feed-forward, RMSNorm
throughout, tensor names as the safetensors files of this architecture carry
them (the reference's GGUF names map onto them one to one:
internal/engine/engine.go:402-433, 921-951)."""
from __future__ import annotations

from ..config.llama import LlamaConfig
from ..model import ModelSpec, Run, token_table
from ..parts.base import PartSpec
from ..registry import register_architecture


def llama_spec(cfg: LlamaConfig) -> ModelSpec:
    position = PartSpec("rope", {
        "head_dim": cfg.head_dim,
        "base": cfg.rope_theta,
        "scaling": cfg.rope_scaling.to_dict() if cfg.rope_scaling else None,
    })
    layers = []
    for i in range(cfg.num_hidden_layers):
        p = f"model.layers.{i}"
        layers.append(PartSpec("prenorm", {
            "mixer": PartSpec("gqa_attention", {
                "width": cfg.hidden_size, "heads": cfg.num_attention_heads,
                "kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
                "position": position, "prefix": p + ".self_attn",
            }),
            "feed_forward": PartSpec("swiglu", {
                "width": cfg.hidden_size, "inner": cfg.intermediate_size, "prefix": p + ".mlp",
            }),
            "mixer_norm": PartSpec("rmsnorm", {
                "width": cfg.hidden_size, "eps": cfg.rms_norm_eps, "name": p + ".input_layernorm.weight",
            }),
            "ffn_norm": PartSpec("rmsnorm", {
                "width": cfg.hidden_size, "eps": cfg.rms_norm_eps,
                "name": p + ".post_attention_layernorm.weight",
            }),
        }))
    return ModelSpec(
        vocab_size=cfg.vocab_size,
        width=cfg.hidden_size,
        embedding=token_table("model.embed_tokens.weight", cfg.vocab_size, cfg.hidden_size),
        layers=tuple(layers),
        schedule=tuple(Run(i) for i in range(cfg.num_hidden_layers)),
        final_norm=PartSpec("rmsnorm", {"width": cfg.hidden_size, "eps": cfg.rms_norm_eps,
                                        "name": "model.norm.weight"}),
        head_name="lm_head.weight",
        tie_head=cfg.tie_word_embeddings,
        stop_ids=tuple(cfg.eos_token_ids),
        bos_id=cfg.bos_token_id,
        max_positions=cfg.max_position_embeddings,
    )


register_architecture("LlamaForCausalLM", LlamaConfig, llama_spec)

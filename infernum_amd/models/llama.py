"""The Llama dense decoder as a ModelSpec: which parts, with which constants, under
which tensor names (infernum-llama/src/graph_builder.rs:201-364 for the names,
:446-536 for the order of operations).
"""
from __future__ import annotations

from ..config.llama import LLAMA_MODEL_TYPES, LlamaConfig
from ..config.registry import register_architecture
from ..parts.base import LayerSpec, ModelSpec, PartSpec, ScheduleEntry


def llama_model_spec(cfg: LlamaConfig, norm_init: tuple = ("ones",), init_std: float = 0.02) -> ModelSpec:
    H, nh, nkv, d = cfg.hidden_size, cfg.num_attention_heads, cfg.num_kv_heads, cfg.head_dim
    position = {
        "kind": "rope",
        "params": {
            "head_dim": d,
            "theta": cfg.rope_theta,
            "scaling": cfg.rope_scaling.to_dict() if cfg.rope_scaling is not None else None,
        },
    }
    layers = []
    for i in range(cfg.num_hidden_layers):
        p = f"model.layers.{i}."
        layers.append(LayerSpec(
            block="prenorm",
            mixer=PartSpec("attention", {
                "hidden_size": H, "num_heads": nh, "num_kv_heads": nkv, "head_dim": d, "position": position,
                "window": cfg.effective_sliding_window(i), "init_std": init_std,
            }, p + "self_attn."),
            feed_forward=PartSpec("swiglu", {
                "hidden_size": H, "intermediate_size": cfg.intermediate_size, "init_std": init_std,
            }, p + "mlp."),
            mixer_norm=PartSpec("rmsnorm", {"size": H, "eps": cfg.rms_norm_eps, "init": norm_init},
                                p + "input_layernorm."),
            feed_forward_norm=PartSpec("rmsnorm", {"size": H, "eps": cfg.rms_norm_eps, "init": norm_init},
                                       p + "post_attention_layernorm."),
        ))
    return ModelSpec(
        vocab_size=cfg.vocab_size,
        hidden_size=H,
        embedding=PartSpec("token", {"vocab_size": cfg.vocab_size, "hidden_size": H, "init_std": init_std},
                           "model.embed_tokens."),
        layers=layers,
        schedule=[ScheduleEntry(i) for i in range(cfg.num_hidden_layers)],
        final_norm=PartSpec("rmsnorm", {"size": H, "eps": cfg.rms_norm_eps, "init": norm_init}, "model.norm."),
        head=PartSpec("linear", {
            "vocab_size": cfg.vocab_size, "hidden_size": H, "fallback": "model.embed_tokens.weight",
            "tied": cfg.tie_word_embeddings, "init_std": init_std,
        }, "lm_head."),
        max_position=cfg.max_position_embeddings,
        bos_token_id=cfg.bos_token_id,
        eos_token_id=cfg.eos_token_id,
    )


for _name in LLAMA_MODEL_TYPES:
    register_architecture(_name, LlamaConfig, llama_model_spec)

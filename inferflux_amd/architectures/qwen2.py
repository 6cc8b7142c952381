"""The Qwen2 / Qwen2.5 dense decoder as a plan of parts.

Per layer, in the reference's order (runtime/backends/cuda/native/transformer_forward.cu:
1676-2712): RMSNorm -> grouped-query attention with q/k/v bias and split-half rotary ->
residual add -> RMSNorm -> SwiGLU -> residual add; after the last layer RMSNorm and the
output head (tied to the embedding table or not).  Tensor names are the Hugging Face ones the
reference resolves (runtime/backends/cuda/native/weight_map.cpp:21-58).
"""
from __future__ import annotations

from ..config.qwen2 import Qwen2Config
from ..config.registry import register_architecture
from ..parts.plan import LayerSpec, ModelPlan, PartSpec, ScheduleEntry


def qwen2_plan(cfg: Qwen2Config) -> ModelPlan:
    H = cfg.hidden_size
    layers = []
    for l in range(cfg.num_hidden_layers):
        p = f"model.layers.{l}"
        layers.append(LayerSpec(
            prefix=p,
            block=PartSpec("prenorm"),
            norm_in=PartSpec("rmsnorm", {"name": f"{p}.input_layernorm", "eps": cfg.rms_norm_eps}),
            mixer=PartSpec("paged_attention", {
                "name": f"{p}.self_attn",
                "n_heads": cfg.num_attention_heads,
                "n_kv_heads": cfg.num_key_value_heads,
                "head_dim": cfg.head_dim,
                "bias": cfg.attention_bias,
                "window": cfg.layer_window(l),
                "position": PartSpec("rotary", {"head_dim": cfg.head_dim, "theta": cfg.rope_theta, "style": "split_half"}),
            }),
            norm_post=PartSpec("rmsnorm", {"name": f"{p}.post_attention_layernorm", "eps": cfg.rms_norm_eps}),
            ffn=PartSpec("swiglu", {"name": f"{p}.mlp", "intermediate_size": cfg.intermediate_size}),
        ))
    return ModelPlan(
        vocab_size=cfg.vocab_size,
        hidden_size=H,
        max_position=cfg.max_position_embeddings,
        embedding=PartSpec("token_embedding", {"name": "model.embed_tokens", "vocab_size": cfg.vocab_size}),
        layers=tuple(layers),
        schedule=tuple(ScheduleEntry(l) for l in range(cfg.num_hidden_layers)),
        final_norm=PartSpec("rmsnorm", {"name": "model.norm", "eps": cfg.rms_norm_eps}),
        lm_head=PartSpec("linear_head", {
            "name": "lm_head", "vocab_size": cfg.vocab_size,
            "tied_to": "model.embed_tokens.weight" if cfg.tie_word_embeddings else None}),
        eos_token_ids=tuple(cfg.eos_token_id),
    )


register_architecture(Qwen2Config, qwen2_plan)

"""The Llama dense decoder as a `ModelSpec`: every layer is pre-norm RMSNorm, grouped-query
attention with rotary encoding over all keys, and a SwiGLU feed-forward
(src/llmserve/model/llama.py:123-185).  Tensor names are the checkpoint's own
(src/llmserve/model/llama.py:3-5): model.embed_tokens, model.layers.N.self_attn.q_proj, ...,
model.norm, lm_head."""

from __future__ import annotations

from ..config.model_config import LLAMA_PRESETS, LlamaConfig
from ..config.registry import register_architecture
from ..parts.spec import LayerSpec, ModelSpec, PartSpec


def llama_spec(cfg: LlamaConfig) -> ModelSpec:
    norm = PartSpec("rmsnorm", {"hidden": cfg.hidden_size, "eps": cfg.rms_norm_eps})
    position = PartSpec("rope", {"head_dim": cfg.head_dim, "theta": cfg.rope_theta})
    mixer = PartSpec("attention", {
        "hidden": cfg.hidden_size, "num_heads": cfg.num_attention_heads,
        "num_kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
        "bias": cfg.attention_bias, "window": None, "position": position})
    feed_forward = PartSpec("swiglu", {"hidden": cfg.hidden_size, "intermediate": cfg.intermediate_size})
    layers = []
    for i in range(cfg.num_hidden_layers):
        p = f"model.layers.{i}."
        layers.append(LayerSpec(
            block="prenorm",
            parts={"mixer": mixer, "feed_forward": feed_forward, "mixer_norm": norm, "feed_forward_norm": norm},
            weights={"mixer": p + "self_attn.", "feed_forward": p + "mlp.",
                     "mixer_norm": p + "input_layernorm.", "feed_forward_norm": p + "post_attention_layernorm."}))
    return ModelSpec(
        hidden_size=cfg.hidden_size, vocab_size=cfg.vocab_size, max_positions=cfg.max_position_embeddings,
        embedding=PartSpec("embedding", {"vocab": cfg.vocab_size, "hidden": cfg.hidden_size}),
        layers=tuple(layers), schedule=tuple(range(cfg.num_hidden_layers)), final_norm=norm,
        head=PartSpec("lm_head", {"vocab": cfg.vocab_size, "hidden": cfg.hidden_size,
                                  "tied": cfg.tie_word_embeddings}),
        weights={"embedding": "model.embed_tokens.", "final_norm": "model.norm.", "head": "lm_head."})


register_architecture("LlamaForCausalLM", LlamaConfig, llama_spec, model_type="llama", presets=LLAMA_PRESETS)

"""Qwen3 dense: configuration -> ModelSpec.

embed -> N x prenorm block( GQA attention with per-head q/k RMSNorm and full-head
neox rotary | SwiGLU MLP ) -> RMSNorm -> lm_head; no biases; weight names as in
models/qwen3/src/model.rs:5-6,427-468,487-496.
"""
from __future__ import annotations

from ..config.qwen3 import Qwen3Config
from ..config.registry import register_architecture
from ..parts.spec import LayerSpec, ModelSpec, RunEntry, part


def build_spec(cfg: Qwen3Config) -> ModelSpec:
    norm = part("rmsnorm", eps=cfg.rms_norm_eps)
    position = part("rotary", theta=cfg.rope_theta, max_positions=cfg.max_position_embeddings, style="neox")
    layers = []
    for i in range(cfg.num_hidden_layers):
        mixer = part("attention", heads=cfg.num_attention_heads, kv_heads=cfg.num_key_value_heads,
                     head_dim=cfg.head_dim, position=position, qk_norm=norm, window=cfg.layer_window(i))
        ff = part("gated_mlp", intermediate=cfg.intermediate_size, act=cfg.hidden_act)
        layers.append(LayerSpec(block=part("prenorm"), mixer=mixer, feed_forward=ff, norm=norm,
                                prefix=f"model.layers.{i}."))
    return ModelSpec(
        architecture=cfg.ARCHITECTURE, vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size,
        max_positions=cfg.max_position_embeddings, layers=layers,
        run=[RunEntry(i) for i in range(cfg.num_hidden_layers)],
        final_norm=norm, final_norm_name="model.norm.", embed_name="model.embed_tokens.weight",
        head_name="lm_head.weight", tie_embeddings=cfg.tie_word_embeddings, eos_token_ids=cfg.eos_token_ids)


register_architecture(Qwen3Config.ARCHITECTURE, Qwen3Config, build_spec)

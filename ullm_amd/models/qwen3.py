"""Qwen3 dense as a plan: every layer is a pre-norm block of grouped-query attention (per-head q/k
norm, rotary positions, optional window) and a SwiGLU feed-forward.

Reference: ullm/models/qwen3.py:133-178 (layer), :199-255 (model), :258-286 (head), tensor names as
bound in :300-336.
"""
from __future__ import annotations

import logging

from ..config.model_config import Qwen3Config
from .model import Choice, ModelPlan
from .registry import register_architecture

logger = logging.getLogger("ullm_amd")


def qwen3_plan(cfg: Qwen3Config) -> ModelPlan:
    layers = []
    windowed = [i for i in range(cfg.num_hidden_layers) if cfg.window_of_layer(i) > 0]
    if windowed:
        # the reference reads none of the sliding-window keys (ullm/models/qwen3.py:48-112 builds every layer
        # with full attention): which layers look back how far is decided here alone
        logger.warning("config.json switches sliding-window attention on (%d of %d layers look back %d keys): the "
                       "reference applies no window, so which layers are windowed and which keys they see is this "
                       "engine's own reading of use_sliding_window / sliding_window / max_window_layers / layer_types",
                       len(windowed), cfg.num_hidden_layers, cfg.sliding_window)
    for i in range(cfg.num_hidden_layers):
        p = f"model.layers.{i}"
        position = Choice("position", "rotary", dict(
            head_dim=cfg.head_dim, theta=cfg.rope_theta, rotary_dim=cfg.head_dim, pairing="half",
            max_positions=None))
        mixer = Choice("mixer", "gqa_attention", dict(
            hidden_size=cfg.hidden_size, num_heads=cfg.num_attention_heads,
            num_kv_heads=cfg.num_key_value_heads, head_dim=cfg.head_dim, prefix=f"{p}.self_attn",
            position=position, qk_norm_eps=cfg.rms_norm_eps, bias=cfg.attention_bias,
            window=cfg.window_of_layer(i)))
        ffn = Choice("ffn", "swiglu", dict(hidden_size=cfg.hidden_size,
                                           intermediate_size=cfg.intermediate_size, prefix=f"{p}.mlp"))
        norm = lambda name: Choice("norm", "rmsnorm", dict(size=cfg.hidden_size, eps=cfg.rms_norm_eps,  # noqa: E731
                                                           weight_name=f"{p}.{name}.weight"))
        layers.append(Choice("block", "prenorm", dict(
            mixer_norm=norm("input_layernorm"), mixer=mixer,
            ffn_norm=norm("post_attention_layernorm"), ffn=ffn)))
    return ModelPlan(
        vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size,
        embedding_weight="model.embed_tokens.weight", layers=layers,
        final_norm=Choice("norm", "rmsnorm", dict(size=cfg.hidden_size, eps=cfg.rms_norm_eps,
                                                  weight_name="model.norm.weight")),
        head_weight="lm_head.weight", tie_head_to_embedding=cfg.tie_word_embeddings,
        init_std=cfg.initializer_range)


register_architecture("Qwen3ForCausalLM", Qwen3Config.from_dict, qwen3_plan)

"""The Llama dense decoder as data: ``LlamaForCausalLM`` -> ModelSpec.

Every layer is a pre-norm block of grouped-query attention with (optionally llama3-scaled)
rotary position encoding and a SwiGLU feed-forward, RMSNorm before each; a final RMSNorm; the
output matrix is the token table when ``tie_word_embeddings`` is set.  Tensor names are the
checkpoint's own (the reference reads the same names, ``base/src/model.cu:69-81``).
"""
from __future__ import annotations

import math
from dataclasses import asdict

from ..config.model_config import LlamaConfig
from ..config.registry import register_architecture
from .spec import LayerSpec, ModelSpec, PartSpec, default_order


def llama_spec(cfg: LlamaConfig) -> ModelSpec:
    rule, params = "plain", None
    if cfg.rope_scaling is not None:
        params = asdict(cfg.rope_scaling)
        rule = params.pop("rope_type")
    position = PartSpec("rotary", dict(head_dim=cfg.head_dim, max_positions=cfg.max_position_embeddings,
                                       theta=cfg.rope_theta, frequencies=rule, frequency_params=params))
    layers = []
    for i in range(cfg.num_hidden_layers):
        p = f"model.layers.{i}."
        layers.append(LayerSpec(
            block=PartSpec("pre_norm"),
            mixer=PartSpec("gqa_attention", dict(
                prefix=p + "self_attn.", hidden_size=cfg.hidden_size,
                num_heads=cfg.num_attention_heads, num_kv_heads=cfg.num_key_value_heads,
                head_dim=cfg.head_dim, scale=1.0 / math.sqrt(cfg.head_dim), position=position)),
            feed_forward=PartSpec("swiglu", dict(
                prefix=p + "mlp.", hidden_size=cfg.hidden_size,
                intermediate_size=cfg.intermediate_size)),
            norms={
                "mixer": PartSpec("rmsnorm", dict(prefix=p + "input_layernorm.", width=cfg.hidden_size,
                                                  eps=cfg.rms_norm_eps)),
                "feed_forward": PartSpec("rmsnorm", dict(prefix=p + "post_attention_layernorm.",
                                                         width=cfg.hidden_size, eps=cfg.rms_norm_eps)),
            },
            prefix=p,
        ))
    return ModelSpec(
        architecture="LlamaForCausalLM",
        hidden_size=cfg.hidden_size,
        vocab_size=cfg.vocab_size,
        embedding_name="model.embed_tokens.weight",
        layers=tuple(layers),
        order=default_order(cfg.num_hidden_layers),
        final_norm=PartSpec("rmsnorm", dict(prefix="model.norm.", width=cfg.hidden_size,
                                            eps=cfg.rms_norm_eps)),
        final_norm_prefix="model.norm.",
        head_name=None if cfg.tie_word_embeddings else "lm_head.weight",
        max_positions=cfg.max_position_embeddings,
        eos_token_ids=cfg.eos_token_id,
        ignorable_tensors=("*.rotary_emb.inv_freq",) + (("lm_head.weight",) if cfg.tie_word_embeddings else ()),
    )


register_architecture("LlamaForCausalLM", LlamaConfig.from_dict, llama_spec, replace=True)

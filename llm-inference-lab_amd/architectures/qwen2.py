"""Qwen2 dense decoder as data: configuration -> ``ModelSpec``.

Tensor names are those of the checkpoint format the reference reads
(rust/engine/src/runner/model/qwen2/engine.rs:291-399); q, k and v carry biases,
the output projection, the feed-forward and the head do not.
"""
from __future__ import annotations

from ..config.qwen2 import Qwen2Config
from ..config.registry import register_architecture
from ..config.spec import BlockSpec, ModelSpec, PartSpec, ScheduleEntry


def build_qwen2_spec(cfg: Qwen2Config) -> ModelSpec:
    blocks = []
    for i in range(cfg.num_hidden_layers):
        p = f"model.layers.{i}."
        mixer = PartSpec(
            "gqa_attention",
            params=dict(
                hidden_size=cfg.hidden_size, num_heads=cfg.num_attention_heads,
                num_kv_heads=cfg.num_key_value_heads, head_dim=cfg.head_dim,
                qkv_bias=True, out_bias=False, window=cfg.layer_window(i),
                position=PartSpec("rope", params=dict(dim=cfg.head_dim, theta=cfg.rope_theta))),
            tensors=dict(
                q_weight=p + "self_attn.q_proj.weight", q_bias=p + "self_attn.q_proj.bias",
                k_weight=p + "self_attn.k_proj.weight", k_bias=p + "self_attn.k_proj.bias",
                v_weight=p + "self_attn.v_proj.weight", v_bias=p + "self_attn.v_proj.bias",
                o_weight=p + "self_attn.o_proj.weight"))
        ffn = PartSpec(
            "swiglu",
            params=dict(hidden_size=cfg.hidden_size, intermediate_size=cfg.intermediate_size,
                        activation=cfg.hidden_act),
            tensors=dict(gate_weight=p + "mlp.gate_proj.weight", up_weight=p + "mlp.up_proj.weight",
                         down_weight=p + "mlp.down_proj.weight"))
        norm = lambda name: PartSpec("rmsnorm", params=dict(size=cfg.hidden_size, eps=cfg.rms_norm_eps),
                                     tensors=dict(weight=p + name + ".weight"))
        blocks.append(BlockSpec("prenorm",
                                parts=dict(norm1=norm("input_layernorm"), mixer=mixer,
                                           norm2=norm("post_attention_layernorm"), feed_forward=ffn),
                                params=dict(hidden_size=cfg.hidden_size)))
    embed_name = "model.embed_tokens.weight"
    head_name = embed_name if cfg.tie_word_embeddings else "lm_head.weight"
    sizes = dict(vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size)
    spec = ModelSpec(
        architecture=Qwen2Config.ARCHITECTURE,
        vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size,
        max_positions=cfg.max_position_embeddings,
        embedding=PartSpec("token_embedding", params=sizes, tensors=dict(weight=embed_name)),
        blocks=tuple(blocks),
        schedule=tuple(ScheduleEntry(i) for i in range(cfg.num_hidden_layers)),
        final_norm=PartSpec("rmsnorm", params=dict(size=cfg.hidden_size, eps=cfg.rms_norm_eps),
                            tensors=dict(weight="model.norm.weight")),
        head=PartSpec("linear_head", params=sizes, tensors=dict(weight=head_name)),
        eos_token_ids=tuple(cfg.eos_token_ids))
    spec.validate()
    return spec


# The two-message prompt that the reference's command line writes out for this model
# (rust/engine/examples/qwen2.rs:122-124).
QWEN2_CHAT_TEMPLATE = ("<|im_start|>system\nYou are Qwen, created by Alibaba Cloud. You are a helpful "
                       "assistant.<|im_end|>\n<|im_start|>user\n{prompt}<|im_end|>\n<|im_start|>assistant\n")

register_architecture(Qwen2Config.ARCHITECTURE, Qwen2Config, build_qwen2_spec, replace=True,
                      chat_template=QWEN2_CHAT_TEMPLATE)

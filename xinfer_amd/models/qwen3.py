"""Qwen3 dense as data: the typed config turned into a `ModelSpec`.

Layer composition follows /root/reference/src/models/qwen3.rs:108-134
(input RMSNorm -> attention -> residual add + post-attention RMSNorm -> SwiGLU MLP
-> residual add), tensor names qwen3.rs:41,54,81,93,217,236-245,261,280.
"""
from __future__ import annotations

from ..config.model_config import Qwen3Config
from ..config.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry
from .registry import ModelFamily, register_architecture


def qwen3_spec_for(cfg: Qwen3Config, tensor_names) -> ModelSpec:
    """A checkpoint that holds `embed_tokens.weight` without the `model.` prefix has no prefix
    anywhere and no head of its own: the reference then reads every tensor without the prefix
    and ties the head to the table (embedding checkpoints, qwen3.rs:200-209)."""
    names = set(tensor_names)
    # a configuration that says nothing about biases takes them if the checkpoint has them
    # (attention.rs:472-476, 388-399)
    bias = cfg.attention_bias
    if bias is None:
        bias = any(n.endswith(".self_attn.q_proj.bias") for n in names)
    if "embed_tokens.weight" in names and "model.embed_tokens.weight" not in names:
        return qwen3_spec(cfg, prefix="", tied=True, bias=bias)
    return qwen3_spec(cfg, bias=bias)


def qwen3_spec(cfg: Qwen3Config, prefix: str = "model.", tied=None, bias=None) -> ModelSpec:
    tied = cfg.tie_word_embeddings if tied is None else bool(tied)
    bias = bool(cfg.attention_bias) if bias is None else bool(bias)
    rope_params = dict(head_dim=cfg.head_dim, rotary_dim=cfg.rotary_dim, theta=cfg.rope_theta,
                       max_positions=cfg.positions, interleaved=False)
    rs = cfg.rope_scaling
    if rs is not None and rs.kind != "default":
        rope_params["scaling"] = dict(
            kind=rs.kind, original=rs.original_positions(cfg.max_position_embeddings), factor=rs.factor,
            low_freq_factor=rs.low_freq_factor, high_freq_factor=rs.high_freq_factor, alpha=rs.alpha,
            beta_fast=rs.beta_fast, beta_slow=rs.beta_slow, extrapolation_factor=rs.extrapolation_factor,
            attn_factor=rs.attn_factor)
    rope = PartSpec("rope", rope_params)
    layers = []
    for i in range(cfg.num_hidden_layers):
        layer_prefix = f"{prefix}layers.{i}"
        mixer = PartSpec("attention", dict(
            hidden_size=cfg.hidden_size, num_heads=cfg.num_attention_heads,
            num_kv_heads=cfg.num_key_value_heads, head_dim=cfg.head_dim,
            bias=bias, qk_norm=True, qk_norm_eps=cfg.rms_norm_eps,
            window=cfg.window_of_layer(i), position=rope,
            scale=float(cfg.head_dim) ** -0.5))
        ffn = PartSpec("gated_mlp", dict(
            hidden_size=cfg.hidden_size, intermediate_size=cfg.intermediate_size,
            activation=cfg.hidden_act))
        norm = PartSpec("rmsnorm", dict(dim=cfg.hidden_size, eps=cfg.rms_norm_eps))
        layers.append(LayerSpec(
            prefix=layer_prefix, block="prenorm", mixer=mixer, feed_forward=ffn,
            norms={"input_layernorm": norm, "post_attention_layernorm": norm},       # qwen3.rs:81,93
            mixer_name="self_attn", feed_forward_name="mlp"))                         # qwen3.rs:41,54
    return ModelSpec(
        architecture=cfg.architecture,
        vocab_size=cfg.vocab_size,
        hidden_size=cfg.hidden_size,
        max_positions=cfg.positions,
        embedding=PartSpec("embedding", dict(
            name=f"{prefix}embed_tokens.weight", vocab_size=cfg.vocab_size, dim=cfg.hidden_size)),
        layers=tuple(layers),
        schedule=tuple(ScheduleEntry(i) for i in range(cfg.num_hidden_layers)),
        final_norm=PartSpec("rmsnorm", dict(
            dim=cfg.hidden_size, eps=cfg.rms_norm_eps, name=f"{prefix}norm.weight")),
        head=PartSpec("lm_head", dict(
            name=f"{prefix}embed_tokens.weight" if tied else "lm_head.weight",
            tied=tied, vocab_size=cfg.vocab_size, dim=cfg.hidden_size)),
        eos_token_ids=tuple(cfg.eos_token_id or ()),
    )


# ChatML, the form Qwen3's own template reduces to for plain system/user/assistant turns
CHATML = ("{% for message in messages %}<|im_start|>{{ message.role }}\n{{ message.content }}<|im_end|>\n{% endfor %}"
          "{% if add_generation_prompt %}<|im_start|>assistant\n{% endif %}")

QWEN3 = ModelFamily("qwen3", Qwen3Config, qwen3_spec, qwen3_spec_for, chat_template=CHATML)
# The reference maps all of these names to ModelType::Qwen3 (utils/mod.rs:2357-2365);
# only the Qwen3 name is registered here because Qwen2 differs (bias, no q/k norm).
register_architecture("Qwen3ForCausalLM", QWEN3)

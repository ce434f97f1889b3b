"""The Qwen3 dense decoder as data: how its configuration becomes a :class:`ModelSpec`.

Layer make-up and tensor names as the reference binds them (src/qwen.cc:77-84 for the three
global tensors, src/qwen.cc:285-308 for the eleven of a layer): pre-norm residual blocks of
grouped-query attention (per-head RMSNorm on q and k, rotary embedding) and a SwiGLU
feed-forward; the head shares the embedding table when ``tie_word_embeddings`` is set or, as
in the reference (src/qwen.cc:80-84), when the checkpoint has no ``lm_head.weight``.
"""
from __future__ import annotations

from ..config.model_config import Qwen3Config
from ..config.registry import ARCHITECTURES, Architecture
from ..config.specs import ModelSpec, PartSpec, RunEntry, prenorm_layer


def qwen3_layer_names(i: int):
    p = f"model.layers.{i}."
    return {
        "mixer.q_proj": p + "self_attn.q_proj.weight",
        "mixer.k_proj": p + "self_attn.k_proj.weight",
        "mixer.v_proj": p + "self_attn.v_proj.weight",
        "mixer.o_proj": p + "self_attn.o_proj.weight",
        "mixer.q_norm.weight": p + "self_attn.q_norm.weight",
        "mixer.k_norm.weight": p + "self_attn.k_norm.weight",
        "feed_forward.gate_proj": p + "mlp.gate_proj.weight",
        "feed_forward.up_proj": p + "mlp.up_proj.weight",
        "feed_forward.down_proj": p + "mlp.down_proj.weight",
        "mixer_norm.weight": p + "input_layernorm.weight",
        "feed_forward_norm.weight": p + "post_attention_layernorm.weight",
    }


def qwen3_model_spec(cfg: Qwen3Config) -> ModelSpec:
    norm = PartSpec("rms", {"size": cfg.hidden_size, "eps": cfg.rms_norm_eps})
    head_norm = PartSpec("rms", {"size": cfg.head_dim, "eps": cfg.rms_norm_eps})
    rotary = PartSpec("rotary", {"rotary_dim": cfg.head_dim, "theta": cfg.rope_theta,
                                 "max_positions": cfg.max_position_embeddings})
    feed_forward = PartSpec("gated_mlp", {"hidden_size": cfg.hidden_size,
                                          "intermediate_size": cfg.intermediate_size,
                                          "activation": cfg.hidden_act})
    layers = []
    for i in range(cfg.num_hidden_layers):
        sliding = cfg.layer_types[i] == "sliding_attention"
        mixer = PartSpec("attention", {
            "hidden_size": cfg.hidden_size, "num_heads": cfg.num_attention_heads,
            "num_kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
            "scale": cfg.head_dim ** -0.5, "qk_norm": head_norm, "position": rotary,
            "window": cfg.sliding_window if sliding else None})
        layers.append(prenorm_layer(mixer, feed_forward, norm, norm, qwen3_layer_names(i)))
    return ModelSpec(
        hidden_size=cfg.hidden_size, vocab_size=cfg.vocab_size,
        embedding_name="model.embed_tokens.weight", layers=layers,
        run_order=[RunEntry(i) for i in range(cfg.num_hidden_layers)],
        final_norm=norm, final_norm_names={"weight": "model.norm.weight"},
        head_name=None if cfg.tie_word_embeddings else "lm_head.weight",
        init_std=cfg.initializer_range, max_positions=cfg.max_position_embeddings)


ARCHITECTURES.register("Qwen3ForCausalLM", Architecture(
    name="Qwen3ForCausalLM", read_config=Qwen3Config.from_dict, model_spec=qwen3_model_spec))

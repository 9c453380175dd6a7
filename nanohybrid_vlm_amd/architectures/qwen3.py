"""The Qwen3 dense decoder as a recipe of parts (nanovllm/models/qwen3.py:120-216).

Nothing here computes: it turns ``Qwen3Config`` into a ``ModelSpec`` and lists the
checkpoint's tensor names with the place each takes in the model's (packed)
parameters (nanovllm/models/qwen3.py:187-193, nanovllm/layers/linear.py:102-108,150-167).
"""
from __future__ import annotations

from ..config.model_config import Qwen3Config
from ..config.registry import Architecture, WeightSource, register_architecture
from ..parts.model import LayerSpec, ModelSpec


def build_spec(cfg: Qwen3Config) -> ModelSpec:
    norm = {"kind": "rmsnorm", "size": cfg.hidden_size, "eps": cfg.rms_norm_eps}
    layer = LayerSpec(
        mixer={
            "kind": "gqa_attention",
            "hidden_size": cfg.hidden_size,
            "num_heads": cfg.num_attention_heads,
            "num_kv_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim,
            "scale": cfg.head_dim ** -0.5,                                   # qwen3.py:39
            # per-head norms of q and k exist only without bias (qwen3.py:68-70)
            "qk_norm_eps": None if cfg.attention_bias else cfg.rms_norm_eps,
            "qkv_bias": cfg.attention_bias,
            "window": None,                                                  # the reference reads no window key
        },
        feed_forward={"kind": "swiglu", "hidden_size": cfg.hidden_size, "intermediate_size": cfg.intermediate_size},
        norm=norm,
        block={"kind": "prenorm"},
        position="default",
    )
    return ModelSpec(
        vocab_size=cfg.vocab_size,
        hidden_size=cfg.hidden_size,
        layers=[layer for _ in range(cfg.num_hidden_layers)],
        final_norm=norm,
        # full rotation: rotary_dim = head_dim (qwen3.py:58)
        positions={"default": {"kind": "rope", "rotary_dim": cfg.head_dim, "base": cfg.rope_theta}},
        max_position=cfg.max_position_embeddings,
        tie_embeddings=cfg.tie_word_embeddings,
    )


def checkpoint_names(cfg: Qwen3Config) -> dict[str, WeightSource]:
    q = cfg.num_attention_heads * cfg.head_dim
    kv = cfg.num_key_value_heads * cfg.head_dim
    inter = cfg.intermediate_size
    names = {"model.embed_tokens.weight": WeightSource("embed.weight"),
             "model.norm.weight": WeightSource("final_norm.weight")}
    if not cfg.tie_word_embeddings:
        names["lm_head.weight"] = WeightSource("head.weight")
    for i in range(cfg.num_hidden_layers):
        src, dst = f"model.layers.{i}.", f"layers.{i}."
        names[src + "input_layernorm.weight"] = WeightSource(dst + "mixer_norm.weight")
        names[src + "post_attention_layernorm.weight"] = WeightSource(dst + "feed_forward_norm.weight")
        kinds = ("weight", "bias") if cfg.attention_bias else ("weight",)
        for kind in kinds:
            names[src + f"self_attn.q_proj.{kind}"] = WeightSource(dst + f"mixer.qkv.{kind}", 0, q)
            names[src + f"self_attn.k_proj.{kind}"] = WeightSource(dst + f"mixer.qkv.{kind}", q, kv)
            names[src + f"self_attn.v_proj.{kind}"] = WeightSource(dst + f"mixer.qkv.{kind}", q + kv, kv)
        names[src + "self_attn.o_proj.weight"] = WeightSource(dst + "mixer.o.weight")
        if not cfg.attention_bias:
            names[src + "self_attn.q_norm.weight"] = WeightSource(dst + "mixer.q_norm.weight")
            names[src + "self_attn.k_norm.weight"] = WeightSource(dst + "mixer.k_norm.weight")
        names[src + "mlp.gate_proj.weight"] = WeightSource(dst + "feed_forward.gate_up.weight", 0, inter)
        names[src + "mlp.up_proj.weight"] = WeightSource(dst + "feed_forward.gate_up.weight", inter, inter)
        names[src + "mlp.down_proj.weight"] = WeightSource(dst + "feed_forward.down.weight")
    return names


def optional_names(cfg: Qwen3Config) -> set[str]:
    # a tied checkpoint may or may not repeat the embedding as lm_head.weight
    return {"lm_head.weight"} if cfg.tie_word_embeddings else set()


QWEN3 = Architecture(
    name="Qwen3ForCausalLM",
    model_types=("qwen3",),
    parse_config=Qwen3Config.from_dict,
    build_spec=build_spec,
    checkpoint_names=checkpoint_names,
    optional_names=optional_names,
)
register_architecture(QWEN3, replace=True)

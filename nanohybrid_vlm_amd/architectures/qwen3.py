"""The Qwen3 dense decoder as a recipe of parts (nanovllm/models/qwen3.py:120-216).

Nothing here computes. ``Qwen3Config`` reads the keys of config.json that the
reference reads on this path, with its defaults for absent keys
(nanovllm/models/qwen3.py:128-144,169-171,201-202 for the layer sizes,
nanovllm/models/registry.py:69-95 for ``model_type`` and ``architectures``,
nanovllm/engine/llm_engine.py:207-223 for ``eos_token_id``); ``build_spec`` turns it
into a ``ModelSpec``; ``checkpoint_names`` lists the checkpoint's tensor names with
the place each takes in the model's (packed) parameters
(nanovllm/models/qwen3.py:187-193, nanovllm/layers/linear.py:102-108,150-167);
``SHAPES`` names the sizes of the family that measurements use.
"""
from __future__ import annotations

from dataclasses import dataclass, field, fields
from typing import Any

from ..config.model_config import ConfigError, require
from ..config.registry import Architecture, WeightSource, register_architecture
from ..parts.model import LayerSpec, ModelSpec


@dataclass(frozen=True)
class Qwen3Config:
    """The Qwen3 dense decoder's own keys (nanovllm/models/qwen3.py:128-144)."""

    architectures: tuple[str, ...]
    model_type: str
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    max_position_embeddings: int
    rms_norm_eps: float
    rope_theta: float
    attention_bias: bool
    hidden_act: str
    tie_word_embeddings: bool
    eos_token_id: int | None = None
    torch_dtype: str | None = None
    raw: dict = field(default_factory=dict, compare=False, repr=False)

    @classmethod
    def from_dict(cls, raw: dict[str, Any]) -> "Qwen3Config":
        hidden = require(raw, "hidden_size")
        heads = require(raw, "num_attention_heads")
        # head_dim defaults to hidden_size // heads (qwen3.py:36,134)
        head_dim = raw.get("head_dim") or hidden // heads
        # attention_bias defaults to True when absent (qwen3.py:133)
        bias = raw.get("attention_bias", True)
        # rope_theta defaults to 1e6 (qwen3.py:135); of rope_scaling only its
        # own "rope_theta" is read (qwen3.py:54-55)
        theta = raw.get("rope_theta", 1000000)
        scaling = raw.get("rope_scaling")
        if isinstance(scaling, dict):
            theta = scaling.get("rope_theta", theta)
        eos = raw.get("eos_token_id")
        if isinstance(eos, (list, tuple)):
            # nanovllm/engine/llm_engine.py:207-223 refuses several end tokens
            raise ConfigError("config.json: a list of eos_token_id is not supported")
        cfg = cls(
            architectures=tuple(raw.get("architectures") or ()),
            model_type=str(raw.get("model_type", "")),
            vocab_size=require(raw, "vocab_size"),
            hidden_size=hidden,
            intermediate_size=require(raw, "intermediate_size"),
            num_hidden_layers=require(raw, "num_hidden_layers"),
            num_attention_heads=heads,
            num_key_value_heads=int(raw.get("num_key_value_heads") or heads),
            head_dim=int(head_dim),
            max_position_embeddings=require(raw, "max_position_embeddings"),
            rms_norm_eps=require(raw, "rms_norm_eps", float),
            rope_theta=float(theta),
            attention_bias=bool(bias),
            hidden_act=str(raw.get("hidden_act", "silu")),
            tie_word_embeddings=bool(raw.get("tie_word_embeddings", False)),
            eos_token_id=None if eos is None else int(eos),
            torch_dtype=raw.get("dtype") or raw.get("torch_dtype"),
            raw=dict(raw),
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        for f in fields(self):
            v = getattr(self, f.name)
            if f.name in ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                          "num_attention_heads", "num_key_value_heads", "head_dim",
                          "max_position_embeddings") and v <= 0:
                raise ConfigError(f"config.json: '{f.name}' must be positive, got {v}")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"config.json: num_attention_heads ({self.num_attention_heads}) is not a multiple of "
                f"num_key_value_heads ({self.num_key_value_heads})")
        if self.head_dim % 2:
            raise ConfigError(f"config.json: head_dim ({self.head_dim}) must be even for the rotation")
        if self.hidden_act != "silu":
            # the reference asserts the same (qwen3.py:110)
            raise ConfigError(f"config.json: hidden_act '{self.hidden_act}' is not supported (only 'silu')")
        if not (self.rms_norm_eps > 0):
            raise ConfigError(f"config.json: rms_norm_eps must be positive, got {self.rms_norm_eps}")

    def to_dict(self) -> dict:
        """The keys as they are written into a config.json."""
        out = {
            "architectures": list(self.architectures),
            "model_type": self.model_type,
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "max_position_embeddings": self.max_position_embeddings,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "attention_bias": self.attention_bias,
            "hidden_act": self.hidden_act,
            "tie_word_embeddings": self.tie_word_embeddings,
            "torch_dtype": self.torch_dtype or "bfloat16",
        }
        if self.eos_token_id is not None:
            out["eos_token_id"] = self.eos_token_id
        return out




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
        eos_token_id=cfg.eos_token_id,
    )


def checkpoint_names(cfg: Qwen3Config) -> dict[str, WeightSource]:
    q = cfg.num_attention_heads * cfg.head_dim
    kv = cfg.num_key_value_heads * cfg.head_dim
    inter = cfg.intermediate_size
    names = {"model.embed_tokens.weight": WeightSource("embed.weight"),
             "model.norm.weight": WeightSource("final_norm.weight")}
    if cfg.tie_word_embeddings:
        # the head's storage is the embedding's (qwen3.py:202-203): a file may repeat it under the head's name
        names["lm_head.weight"] = WeightSource("embed.weight", copy=True)
    else:
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


def _shape(layers, hidden, heads, kv_heads, head_dim, inter, vocab=151936, theta=1000000.0, eps=1e-6, tie=False,
           max_pos=40960):
    return {
        "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "num_hidden_layers": layers,
        "hidden_size": hidden, "num_attention_heads": heads, "num_key_value_heads": kv_heads, "head_dim": head_dim,
        "intermediate_size": inter, "vocab_size": vocab, "rope_theta": theta, "rms_norm_eps": eps,
        "tie_word_embeddings": tie, "max_position_embeddings": max_pos, "attention_bias": False, "hidden_act": "silu",
        "eos_token_id": 151645 if vocab > 151645 else 0, "torch_dtype": "bfloat16",
    }


# config.json contents of the sizes that measurements and examples name; the engine itself takes every size
# from a config.json
SHAPES = {
    "tinyA": _shape(2, 64, 4, 2, 16, 128, vocab=256, theta=10000.0, eps=1e-6, tie=True, max_pos=128),
    "tinyB": _shape(3, 96, 6, 1, 32, 160, vocab=389, theta=1000000.0, eps=1e-5, tie=False, max_pos=256),
    "0.6b": _shape(28, 1024, 16, 8, 128, 3072, tie=True),
    "1.7b": _shape(28, 2048, 16, 8, 128, 6144, tie=True),
    "4b": _shape(36, 2560, 32, 8, 128, 9728, tie=True),
    "8b": _shape(36, 4096, 32, 8, 128, 12288),
    "14b": _shape(40, 5120, 40, 8, 128, 17408),
    "32b": _shape(64, 5120, 64, 8, 128, 25600),
}


QWEN3 = Architecture(
    name="Qwen3ForCausalLM",
    model_types=("qwen3",),
    parse_config=Qwen3Config.from_dict,
    build_spec=build_spec,
    checkpoint_names=checkpoint_names,
    named_shapes=SHAPES,
)
register_architecture(QWEN3, replace=True)

"""Typed model configuration read from a checkpoint's ``config.json``.

Every size and constant of the model comes from here; no part of the engine
carries a default of its own for something ``config.json`` can say.

The keys, and the defaults for absent keys, are the ones the reference reads on
its Qwen3 path: nanovllm/models/qwen3.py:128-144,169-171,201-202 (layer sizes),
nanovllm/models/registry.py:69-95 (``model_type``, ``architectures``),
nanovllm/engine/llm_engine.py:207-223 (``eos_token_id``).
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field, fields
from typing import Any


class ConfigError(ValueError):
    """A config.json that the engine cannot run, with the key that is at fault."""


def _require(raw: dict, key: str, kind=int):
    if key not in raw or raw[key] is None:
        raise ConfigError(f"config.json: required key '{key}' is missing")
    value = raw[key]
    if kind is int and (isinstance(value, bool) or not isinstance(value, int)):
        raise ConfigError(f"config.json: '{key}' must be an integer, got {value!r}")
    if kind is float and (isinstance(value, bool) or not isinstance(value, (int, float))):
        raise ConfigError(f"config.json: '{key}' must be a number, got {value!r}")
    return kind(value)


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
        hidden = _require(raw, "hidden_size")
        heads = _require(raw, "num_attention_heads")
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
            vocab_size=_require(raw, "vocab_size"),
            hidden_size=hidden,
            intermediate_size=_require(raw, "intermediate_size"),
            num_hidden_layers=_require(raw, "num_hidden_layers"),
            num_attention_heads=heads,
            num_key_value_heads=int(raw.get("num_key_value_heads") or heads),
            head_dim=int(head_dim),
            max_position_embeddings=_require(raw, "max_position_embeddings"),
            rms_norm_eps=_require(raw, "rms_norm_eps", float),
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


def read_config_json(folder: str) -> dict:
    path = os.path.join(folder, "config.json")
    if not os.path.isfile(path):
        raise FileNotFoundError(f"no config.json in model folder '{folder}'")
    with open(path) as f:
        raw = json.load(f)
    if not isinstance(raw, dict):
        raise ConfigError(f"{path}: top level must be an object")
    # a multimodal checkpoint nests the decoder's keys (nanovllm/config.py:318-322)
    if "text_config" in raw and isinstance(raw["text_config"], dict) and "hidden_size" not in raw:
        merged = dict(raw["text_config"])
        merged.setdefault("architectures", raw.get("architectures"))
        raw = merged
    return raw

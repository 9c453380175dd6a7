"""Reading a checkpoint's ``config.json``, and the helpers that an architecture's
typed configuration is written with.

Every size and constant of a model comes from its config.json; no part of the
engine carries a default of its own for something config.json can say. Which keys
an architecture reads, and the defaults for absent ones, is that architecture's
own affair (``architectures/``): this module knows no architecture.
"""
from __future__ import annotations

import json
import os


class ConfigError(ValueError):
    """A config.json that the engine cannot run, with the key that is at fault."""


def require(raw: dict, key: str, kind=int):
    """``raw[key]`` as ``kind`` (int or float); a missing key or a value of another kind is a ``ConfigError``."""
    if key not in raw or raw[key] is None:
        raise ConfigError(f"config.json: required key '{key}' is missing")
    value = raw[key]
    if kind is int and (isinstance(value, bool) or not isinstance(value, int)):
        raise ConfigError(f"config.json: '{key}' must be an integer, got {value!r}")
    if kind is float and (isinstance(value, bool) or not isinstance(value, (int, float))):
        raise ConfigError(f"config.json: '{key}' must be a number, got {value!r}")
    return kind(value)


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

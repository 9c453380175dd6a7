"""Random weights: a model folder (config.json, model.safetensors) from a
configuration and a seed. The reference has no such mode.

Matrices, embeddings and biases are N(0, 0.02^2); norm weights are 1 + N(0, 0.1^2).
Every tensor is drawn in float32 from a generator seeded with (seed, position of
the tensor in the architecture's name table), then cast to the stored element
type, so a float32 and a bfloat16 folder of one seed hold the same numbers up to
rounding and a tensor's values do not depend on the other tensors.
"""
from __future__ import annotations

import json
import os

import torch

from ..config.registry import resolve_architecture

_STORE = {"bfloat16": torch.bfloat16, "float32": torch.float32}


def _draw(init: str, shape, gen: torch.Generator) -> torch.Tensor:
    if init == "norm":
        return 1.0 + 0.1 * torch.randn(shape, generator=gen, dtype=torch.float32)
    if init in ("normal", "zeros"):
        # biases are "zeros" at a fresh initialisation; random ones test more
        return 0.02 * torch.randn(shape, generator=gen, dtype=torch.float32)
    raise ValueError(f"unknown initialisation '{init}'")


def random_checkpoint_tensors(raw_config: dict, seed: int, store_dtype: str = "bfloat16") -> dict[str, torch.Tensor]:
    """The checkpoint's tensors by their checkpoint names (CPU)."""
    from ..parts.model import DecoderModel

    arch = resolve_architecture(raw_config)
    cfg = arch.parse_config(raw_config)
    model = DecoderModel(arch.build_spec(cfg))
    specs = model.all_param_specs()
    out = {}
    for index, (name, src) in enumerate(arch.checkpoint_names(cfg).items()):
        if src.copy:                                   # what a file may repeat is written once
            continue
        spec = specs[src.param]
        shape = ((src.rows,) + tuple(spec.shape[1:])) if src.rows is not None else tuple(spec.shape)
        gen = torch.Generator(device="cpu")
        gen.manual_seed((int(seed) * 1000003 + index) & 0x7FFFFFFFFFFFFFFF)
        out[name] = _draw(spec.init, shape, gen).to(_STORE[store_dtype])
    return out


def write_random_model(folder: str, raw_config: dict, seed: int, store_dtype: str = "bfloat16") -> str:
    """Writes ``config.json`` and ``model.safetensors`` into ``folder`` and returns it."""
    from safetensors.torch import save_file

    if store_dtype not in _STORE:
        raise ValueError(f"store_dtype must be one of {sorted(_STORE)}")
    os.makedirs(folder, exist_ok=True)
    arch = resolve_architecture(raw_config)
    cfg = arch.parse_config(raw_config)            # refuses a bad configuration before anything is written
    config_out = dict(raw_config)
    config_out.setdefault("architectures", [arch.name])
    config_out["torch_dtype"] = store_dtype
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(config_out, f, indent=2)
    tensors = random_checkpoint_tensors(raw_config, seed, store_dtype)
    save_file(tensors, os.path.join(folder, "model.safetensors"), metadata={"format": "pt"})
    return folder


def fill_from_device_generator(model, seed: int, dtype: torch.dtype, device) -> dict[str, torch.Tensor]:
    """The same distributions drawn straight into the model's parameters on the
    device by the device's own generator, for measurements at sizes whose files would take
    minutes to write. These are other numbers than ``write_random_model`` writes for the same
    seed (another generator, one stream for all tensors): a model made this way is compared with
    nothing but itself."""
    gen = torch.Generator(device=device)
    gen.manual_seed(int(seed))
    params = {}
    for name, spec in model.all_param_specs().items():
        # what a checkpoint would store in 32-bit (norm weights, routers) stays float32 here too
        t = torch.empty(spec.shape, dtype=torch.float32 if spec.keeps_float32 else dtype, device=device)
        if spec.init == "norm":
            t.normal_(1.0, 0.1, generator=gen)
        else:
            t.normal_(0.0, 0.02, generator=gen)
        params[name] = t
    model.bind_all(params)
    return params


def build_random_model(raw_config: dict, seed: int, dtype: str | torch.dtype = "bfloat16", device="cuda:0",
                       options: dict | None = None):
    """(architecture, typed configuration, model with random weights bound) from config.json contents: what
    ``ModelRunner`` and ``LLM`` take in place of a model folder. The weights are drawn on the device
    (``fill_from_device_generator``: not the numbers that a folder of the same seed holds).
    ``options``: engine options offered to the parts' constructors (see ``DecoderModel``)."""
    from ..parts.model import DecoderModel

    arch = resolve_architecture(raw_config)
    cfg = arch.parse_config(raw_config)
    model = DecoderModel(arch.build_spec(cfg), options=options)
    if isinstance(dtype, str):
        dtype = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32}[dtype]
    fill_from_device_generator(model, seed, dtype, device)
    return arch, cfg, model

"""Small helpers shared by the tests."""
from __future__ import annotations

import os

import torch

# Largest allowed difference between the engine's logits and the plain float32 implementation's (same stored
# weights), as a fraction of the standard deviation of the plain logits (0.17 to 0.19 for the tiny models, 0.45
# for the one with 512 channels): an absolute bound would mean something else for every model.
#   float32: both sides round only in float32; observed 3e-6 / 0.19 = 2e-5 of the deviation at most.
#   bfloat16: activations are rounded to 8 significant bits after every kernel; through 2-3 layers that gives
#   0.025 to 0.05 of the deviation (4e-3 .. 9e-3 for the tiny models, 2.2e-2 at 512 channels).
RELATIVE_TOLERANCE = {"float32": 1e-4, "bfloat16": 1e-1}
# the same as absolute numbers for the tiny models A, B, C (deviation about 0.2), where a test has no plain logits at hand
TOLERANCE = {"float32": 2e-5, "bfloat16": 2e-2}


def tolerance_for(dtype: str, plain_logits) -> float:
    """``plain_logits``: tensor or dict of tensors of the plain implementation."""
    import torch
    if isinstance(plain_logits, dict):
        plain_logits = torch.cat([t.reshape(-1) for t in plain_logits.values()])
    return RELATIVE_TOLERANCE[dtype] * plain_logits.float().std().item()


def sharpen(folder: str, out_folder: str, factor: float = 2.0) -> str:
    """A copy of a model folder whose q and k norm weights are ``factor`` times larger:
    attention scores grow by factor^2, so single keys stand out and a key that is
    lost or read from the wrong place changes the result visibly."""
    import shutil
    from safetensors.torch import load_file, save_file

    os.makedirs(out_folder, exist_ok=True)
    shutil.copy(os.path.join(folder, "config.json"), os.path.join(out_folder, "config.json"))
    tensors = load_file(os.path.join(folder, "model.safetensors"))
    for name in tensors:
        if name.endswith("q_norm.weight") or name.endswith("k_norm.weight"):
            tensors[name] = (tensors[name].float() * factor).to(tensors[name].dtype)
    save_file(tensors, os.path.join(out_folder, "model.safetensors"), metadata={"format": "pt"})
    return out_folder


def max_abs_diff(a: torch.Tensor, b: torch.Tensor) -> float:
    return (a.float() - b.float()).abs().max().item()


def first_difference(a: torch.Tensor, b: torch.Tensor, tol: float) -> str:
    """Names the first position whose logits differ by more than ``tol``."""
    bad = ((a.float() - b.float()).abs() > tol).any(dim=-1).nonzero()
    if bad.numel() == 0:
        return "no difference"
    return f"first wrong position {int(bad[0])} of {a.shape[0]} (max diff there {max_abs_diff(a[bad[0]], b[bad[0]]):.3e})"

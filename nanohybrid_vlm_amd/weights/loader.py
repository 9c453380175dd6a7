"""Weights from safetensors files, placed by tensor name.

Every ``*.safetensors`` file of the folder is read (sorted; no index file is
consulted, as in nanovllm/utils/loader.py:33-46). The architecture's table says
where each checkpoint tensor goes: whole into a parameter, or as a band of rows of
a packed one (q | k | v, gate | up). All faults are found before anything is
copied and are reported together in one error: tensors the model does not know,
tensors it needs and did not get, and tensors of the wrong shape
(nanovllm/utils/loader.py:231-273 raises its three lists the same way).

Element types: a 16-bit tensor becomes bfloat16 (float32 in a float32 run);
a tensor stored in 32-bit stays float32 if the parameter allows it (norm weights),
integer tables become int32.
"""
from __future__ import annotations

import glob
import os

import torch
from safetensors import safe_open


class WeightsError(RuntimeError):
    """One error for everything that is wrong with a checkpoint."""

    def __init__(self, folder, unexpected, missing, wrong_shape, differing=()):
        self.unexpected = list(unexpected)
        self.missing = list(missing)
        self.wrong_shape = list(wrong_shape)
        self.differing = list(differing)
        lines = [f"the checkpoint in '{folder}' does not fit the model:"]
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.wrong_shape:
            lines.append(f"  wrong shapes ({len(self.wrong_shape)}): " + "; ".join(self.wrong_shape))
        if self.differing:
            lines.append(f"  copies that differ from the tensor they repeat ({len(self.differing)}): "
                         + "; ".join(self.differing))
        super().__init__("\n".join(lines))


_ST_DTYPES_32 = {"F32", "F64"}
_ST_DTYPES_INT = {"I8", "I16", "I32", "I64", "U8", "U16", "U32", "U64", "BOOL"}


def _files(folder: str) -> list[str]:
    files = sorted(glob.glob(os.path.join(folder, "*.safetensors")))
    if not files:
        raise FileNotFoundError(f"no *.safetensors file in model folder '{folder}'")
    return files


def load_weights(model, arch, cfg, folder: str, dtype: torch.dtype, device) -> dict[str, torch.Tensor]:
    """Allocates the model's parameters on ``device``, fills them from the folder
    and binds them to the model's parts. Returns the parameters by name."""
    specs = model.all_param_specs()
    sources = arch.checkpoint_names(cfg)
    for name, src in sources.items():
        if src.param not in specs:
            raise KeyError(f"architecture '{arch.name}' maps '{name}' to unknown parameter '{src.param}'")

    # pass 1: names, shapes and stored element types, nothing is read yet
    unexpected, wrong_shape = [], []
    found: dict[str, tuple[str, str]] = {}           # checkpoint name -> (file, stored dtype)
    for path in _files(folder):
        with safe_open(path, framework="pt", device="cpu") as f:
            for key in f.keys():
                if any(key.startswith(p) for p in arch.ignored_prefixes):
                    continue
                if key not in sources:
                    unexpected.append(key)
                    continue
                sl = f.get_slice(key)
                shape = tuple(sl.get_shape())
                src = sources[key]
                pshape = specs[src.param].shape
                want = ((src.rows,) + tuple(pshape[1:])) if src.rows is not None else tuple(pshape)
                if shape != want:
                    wrong_shape.append(f"{key}: stored {list(shape)}, needed {list(want)}")
                found[key] = (path, sl.get_dtype())
    missing = [name for name, src in sources.items() if name not in found and not src.copy]
    # a stored copy (a tied head beside the embedding) must repeat its original: the reference copies it into the
    # shared storage (nanovllm/models/qwen3.py:202-203), so a differing copy would silently replace the embedding
    differing = []
    originals = {(src.param, src.row_start, src.rows): name for name, src in sources.items() if not src.copy}
    for name, src in sources.items():
        if src.copy and name in found and not wrong_shape:
            original = originals.get((src.param, src.row_start, src.rows))
            if original is None or original not in found:
                continue
            with safe_open(found[name][0], framework="pt", device="cpu") as f:
                a = f.get_tensor(name)
            with safe_open(found[original][0], framework="pt", device="cpu") as f:
                b = f.get_tensor(original)
            if a.shape != b.shape or not torch.equal(a.to(torch.float32), b.to(torch.float32)):
                differing.append(f"{name} is not equal to {original}")
            del a, b
    if unexpected or missing or wrong_shape or differing:
        raise WeightsError(folder, sorted(unexpected), missing, wrong_shape, differing)

    # element type of every parameter
    params: dict[str, torch.Tensor] = {}
    by_param: dict[str, list[str]] = {}
    for name, src in sources.items():
        if name in found and not src.copy:
            by_param.setdefault(src.param, []).append(name)
    for pname, spec in specs.items():
        stored = {found[n][1] for n in by_param.get(pname, [])}
        if stored and stored <= _ST_DTYPES_INT:
            pdtype = torch.int32
        elif spec.keeps_float32 and stored and stored <= _ST_DTYPES_32:
            pdtype = torch.float32
        else:
            pdtype = dtype
        params[pname] = torch.empty(spec.shape, dtype=pdtype, device=device)

    # pass 2: copy, file by file
    by_file: dict[str, list[str]] = {}
    for name, (path, _) in found.items():
        if not sources[name].copy:                       # (a copy was compared with its original above)
            by_file.setdefault(path, []).append(name)
    for path, names in by_file.items():
        with safe_open(path, framework="pt", device="cpu") as f:
            for name in names:
                src = sources[name]
                target = params[src.param]
                if src.rows is not None:
                    target = target.narrow(0, src.row_start, src.rows)
                target.copy_(f.get_tensor(name))
    model.bind_all(params)
    return params

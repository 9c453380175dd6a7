"""Plain, slow, whole-sequence Qwen3 dense decoder in float32 on the CPU.

This file is the oracle of the test-suite. It has no cache, no batching and no
kernels: every function takes whole sequences and is written from the formulas
of the reference engine, one function per part. It shares no code with the
package under test (it reads ``config.json`` and ``model.safetensors`` itself).

Each function cites the lines of the reference it is written from
(paths relative to the reference's root).
"""
from __future__ import annotations

import json
import math
import os

import torch


# Where an engine that computes in bfloat16 stores a result in bfloat16, ``stored`` rounds it to that type and back;
# by default it does nothing and everything is float32. The reference runs its model in bfloat16 throughout
# (nanovllm/engine/model_runner.py sets the default dtype from the configuration's torch_dtype), so every
# layer's output is rounded there: projections, norms, rotated queries and keys, the attention's output
# (flash-attention also rounds the softmax's weights before the second product), the gated product.
# The residual sum is kept in float32 here, as the rules of this build ask.
_STORED_DTYPE = None


class stored_as:
    """``with stored_as(torch.bfloat16): logits(...)``: the same formulas with stored results rounded."""

    def __init__(self, dtype):
        self.dtype = dtype

    def __enter__(self):
        global _STORED_DTYPE
        self.old, _STORED_DTYPE = _STORED_DTYPE, self.dtype

    def __exit__(self, *exc):
        global _STORED_DTYPE
        _STORED_DTYPE = self.old


def stored(x: torch.Tensor) -> torch.Tensor:
    return x if _STORED_DTYPE is None else x.to(_STORED_DTYPE).to(torch.float32)


def read_model_folder(folder: str):
    """config.json as a dict and every tensor of model.safetensors as float32."""
    from safetensors import safe_open

    with open(os.path.join(folder, "config.json")) as f:
        config = json.load(f)
    tensors = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt", device="cpu") as f:
        for name in f.keys():
            tensors[name] = f.get_tensor(name).to(torch.float32)
    return config, tensors


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """nanovllm/layers/layernorm.py:16-26: mean of squares over the last
    dimension, eps inside the square root, weight multiplied last."""
    x = x.to(torch.float32)
    var = x.pow(2).mean(dim=-1, keepdim=True)
    # (layernorm.py:25: the scaled row goes back to the model's type before the weight is multiplied in)
    return stored(stored(x * torch.rsqrt(var + eps)) * weight)


def add_rms_norm(x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, eps: float):
    """nanovllm/layers/layernorm.py:28-40: the sum is the new residual and the
    norm is taken of that sum."""
    s = x.to(torch.float32) + residual.to(torch.float32)
    return rms_norm(s, weight, eps), s


def rope_angles(positions: torch.Tensor, rotary_dim: int, base: float) -> torch.Tensor:
    """nanovllm/layers/rotary_embedding.py:83-85: inv_freq_j = base^(-2j/d),
    angle[p, j] = p * inv_freq_j, all in float32."""
    inv_freq = 1.0 / (base ** (torch.arange(0, rotary_dim, 2, dtype=torch.float32, device=positions.device) / rotary_dim))
    return positions.to(torch.float32)[:, None] * inv_freq[None, :]


def apply_rope(x: torch.Tensor, positions: torch.Tensor, base: float, rotary_dim: int | None = None) -> torch.Tensor:
    """nanovllm/layers/rotary_embedding.py:6-14: the head is cut into a first
    and a second half; pair (j, j + d/2) is turned by angle[p, j].
    x: [T, heads, D]. Only the first ``rotary_dim`` entries turn
    (nanovllm/models/qwen3.py:58 passes rotary_dim = head_dim)."""
    d = x.shape[-1] if rotary_dim is None else rotary_dim
    ang = rope_angles(positions, d, base)
    cos = ang.cos()[:, None, :]
    sin = ang.sin()[:, None, :]
    xr = x[..., :d].to(torch.float32)
    x1, x2 = xr[..., : d // 2], xr[..., d // 2:]
    y1 = x1 * cos - x2 * sin
    y2 = x2 * cos + x1 * sin
    return stored(torch.cat((y1, y2, x[..., d:].to(torch.float32)), dim=-1))


def causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
                     window: int | None = None) -> torch.Tensor:
    """nanovllm/layers/attention.py:64-74 (flash-attention, causal) and
    nanovllm/models/qwen3.py:39 (scale = head_dim ** -0.5). q: [T, Hq, D],
    k, v: [T, Hkv, D]; query head h reads kv head h // (Hq // Hkv). A query at
    position p sees the keys at 0..p, or p-window+1..p if a window is given."""
    T, Hq, D = q.shape
    Hkv = k.shape[1]
    group = Hq // Hkv
    out = torch.empty(T, Hq, v.shape[-1], dtype=torch.float32, device=q.device)
    pos = torch.arange(T, device=q.device)
    allowed = pos[None, :] <= pos[:, None]
    if window is not None:
        allowed &= pos[None, :] > pos[:, None] - window
    for h in range(Hq):
        kh = k[:, h // group, :].to(torch.float32)
        vh = v[:, h // group, :].to(torch.float32)
        scores = (q[:, h, :].to(torch.float32) @ kh.T) * scale
        scores = scores.masked_fill(~allowed, float("-inf"))
        if _STORED_DTYPE is None:
            out[:, h, :] = torch.softmax(scores, dim=-1) @ vh
        else:
            # the weights are rounded for the second product; their sum is taken before the rounding
            e = torch.exp(scores - scores.max(dim=-1, keepdim=True).values)
            out[:, h, :] = (stored(e) @ vh) / e.sum(dim=-1, keepdim=True)
    return stored(out)


def swiglu(x: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor) -> torch.Tensor:
    """nanovllm/models/qwen3.py:113-117 and nanovllm/layers/activation.py:10-11:
    silu(x Wg^T) * (x Wu^T), then the down projection."""
    g = stored(x @ w_gate.T)
    u = stored(x @ w_up.T)
    return stored(stored(g * torch.sigmoid(g) * u) @ w_down.T)


def attention_block(x: torch.Tensor, positions: torch.Tensor, w: dict, prefix: str, cfg: dict) -> torch.Tensor:
    """nanovllm/models/qwen3.py:77-87: projections, per-head norms of q and k
    (only without bias, :82-84), rotation, attention, output projection."""
    Hq = cfg["num_attention_heads"]
    Hkv = cfg["num_key_value_heads"]
    D = cfg.get("head_dim") or cfg["hidden_size"] // Hq          # qwen3.py:36
    eps = cfg["rms_norm_eps"]
    bias = cfg.get("attention_bias", True)                       # qwen3.py:133
    theta = cfg.get("rope_theta", 1000000)                       # qwen3.py:135
    scaling = cfg.get("rope_scaling")
    if isinstance(scaling, dict):                                # qwen3.py:54-55
        theta = scaling.get("rope_theta", theta)
    T = x.shape[0]
    q = x @ w[prefix + "q_proj.weight"].T
    k = x @ w[prefix + "k_proj.weight"].T
    v = x @ w[prefix + "v_proj.weight"].T
    if bias:
        q = q + w[prefix + "q_proj.bias"]
        k = k + w[prefix + "k_proj.bias"]
        v = v + w[prefix + "v_proj.bias"]
    q, k, v = stored(q), stored(k), stored(v)
    q = q.view(T, Hq, D)
    k = k.view(T, Hkv, D)
    v = v.view(T, Hkv, D)
    if not bias:
        q = rms_norm(q, w[prefix + "q_norm.weight"], eps)
        k = rms_norm(k, w[prefix + "k_norm.weight"], eps)
    q = apply_rope(q, positions, theta)
    k = apply_rope(k, positions, theta)
    o = causal_attention(q, k, v, D ** -0.5)
    return stored(o.reshape(T, Hq * D) @ w[prefix + "o_proj.weight"].T)


def hidden_states(cfg: dict, w: dict, token_ids, first_position: int = 0) -> torch.Tensor:
    """nanovllm/models/qwen3.py:152-159 and :178-182, written as the usual
    pre-norm block: r += attn(norm(r)); r += mlp(norm(r)); final norm."""
    device = w["model.embed_tokens.weight"].device          # (the tensors may be moved to another device as they are)
    ids = torch.as_tensor(token_ids, dtype=torch.long, device=device)
    positions = torch.arange(first_position, first_position + ids.numel(), device=device)
    eps = cfg["rms_norm_eps"]
    assert cfg.get("hidden_act", "silu") == "silu"               # qwen3.py:110
    r = w["model.embed_tokens.weight"][ids]                      # embed_head.py:38
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        x = rms_norm(r, w[p + "input_layernorm.weight"], eps)
        r = r + attention_block(x, positions, w, p + "self_attn.", cfg)
        x = rms_norm(r, w[p + "post_attention_layernorm.weight"], eps)
        r = r + swiglu(x, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    return rms_norm(r, w["model.norm.weight"], eps)


def logits(cfg: dict, w: dict, token_ids, first_position: int = 0) -> torch.Tensor:
    """nanovllm/layers/embed_head.py:61 and nanovllm/models/qwen3.py:202-203:
    logits = h W^T with W the embedding itself when the two are tied.
    Returns [len, vocab] for every position."""
    h = hidden_states(cfg, w, token_ids, first_position)
    head = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings", False) else w["lm_head.weight"]
    return h @ head.T


def greedy_generate(cfg: dict, w: dict, prompt, n_new: int, eos: int | None = None):
    """Greedy decoding by running the whole sequence again for every token
    (nanovllm/layers/sampler.py:17: argmax of the last position's logits;
    nanovllm/engine/scheduler.py:976-983: the end token is kept)."""
    ids = list(prompt)
    out = []
    for _ in range(n_new):
        nxt = int(logits(cfg, w, ids)[-1].argmax())
        ids.append(nxt)
        out.append(nxt)
        if eos is not None and nxt == eos:
            break
    return out


def sample_noise(seed: int, request: int, step: int, n: int) -> torch.Tensor:
    """The engine's own counter-based noise (no counterpart in the reference,
    which draws from torch's global generator, nanovllm/layers/sampler.py:50-54):
    24 bits from a 64-bit mix of (seed, request, step, index), then Exp(1) noise
    ``noise_of_bits``. Written here independently, in Python integers."""
    mask = (1 << 64) - 1

    def mix(z):
        z = (z + 0x9E3779B97F4A7C15) & mask
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & mask
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & mask
        return z ^ (z >> 31)

    key = mix(mix(mix(seed & mask) ^ (request & mask)) ^ (step & mask))
    out = torch.empty(n, dtype=torch.float32)
    for i in range(n):
        out[i] = noise_of_bits(mix(key ^ i) >> 40)      # 24 random bits
    return out


def noise_of_bits(bits: int) -> float:
    """-log(u) with u = (bits + 0.5) / 2^24, the middle of the bucket of the 24 bits, in double precision."""
    return -math.log((bits + 0.5) / 16777216.0)


def sample_token(logits_row: torch.Tensor, temperature: float, noise: torch.Tensor | None) -> int:
    """nanovllm/layers/sampler.py:12-65: argmax when temperature is 0, else
    argmax(softmax(logits / T) / noise) with noise ~ Exp(1) clamped at 1e-10."""
    row = logits_row.to(torch.float32)
    if temperature == 0:
        return int(row.argmax())
    probs = torch.softmax(row / temperature, dim=-1)
    return int((probs / noise.clamp_min(1e-10)).argmax())

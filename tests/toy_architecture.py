"""A toy architecture for the tests, defined here and nowhere in the package: a mixer that
keeps state of its own per request (in two versions: one that loops over the step's
requests on the host, and one that works from the step's device tensors alone and can
therefore be recorded into a graph), a feed-forward that routes every token to one of
several experts, a position encoding of its own (other angles, on a part of the head
only, over two position axes: even pairs turn by the first coordinate of a token's
position, odd pairs by the second), a block arrangement of its own with a third norm
after the mixer (of another eps than the layer's other norms), an embedding scale and a
cap on the logits, a layer with a window, a layer that runs twice and an entry that
reads another entry's cache; and its plain whole-sequence computation.

Importing this module registers the parts and the architecture (so the command line can
take it as ``--plugin toy_architecture``); ``unregister()`` takes them out again.
config.json of a toy model: {"architectures": ["ToyForCausalLM"], "model_type": "toy",
"device_state": bool, "no_window": bool, "eos_token_id": int or absent}.
"""
import math

import torch

import plain_qwen3 as plain
from nanohybrid_vlm_amd.config.registry import (Architecture, WeightSource, register_architecture,
                                                unregister_architecture)
from nanohybrid_vlm_amd.parts import BLOCKS, FEED_FORWARDS, MIXERS, POSITION_ENCODINGS, ParamSpec, Part, StateNeed
from nanohybrid_vlm_amd.parts.model import DecoderModel, LayerSpec, ModelSpec, RunEntry

H, HEADS, KV, D, INTER, VOCAB, WINDOW, DECAY = 48, 3, 1, 16, 64, 97, 5, 0.75
EXPERTS, EXPERT_INTER, TOY_ROT, TOY_STEP = 3, 40, 8, 0.05
AXES, EMBED_SCALE, LOGIT_CAP, POST_EPS = 2, 1.75, 4.0, 1e-2


class DecayingSum(Part):
    """Toy mixer with state: s_t = decay * s_(t-1) + x_t per request, output s_t W^T.
    The state of a request lives in its state slot between steps. This version walks over the step's
    requests on the host, so a step with it cannot be recorded."""

    recordable = False

    def __init__(self, hidden_size: int, decay: float, position=None):
        self.hidden_size, self.decay = hidden_size, decay

    def param_specs(self):
        return {"out.weight": ParamSpec((self.hidden_size, self.hidden_size))}

    def bind(self, params):
        self.weight = params["out.weight"]

    def cache_need(self):
        return StateNeed({"sum": ((self.hidden_size,), torch.float32)})

    def forward(self, x, step, cache):
        pool = cache.state["sum"]
        out = torch.empty_like(x)
        t = 0
        for start, n, slot in zip(step.host["starts"], step.host["q_lens"], step.host["state_slots"]):
            s = torch.zeros_like(pool[slot]) if start == 0 else pool[slot].clone()   # a new request starts from zero
            for i in range(n):
                s = self.decay * s + x[t + i].float()
                out[t + i] = (s @ self.weight.float().T).to(x.dtype)
            pool[slot] = s
            t += n
        return out


class DecayingSumOnDevice(DecayingSum):
    """The same mixer from the step's device tensors alone, with the same launches whatever they hold:
    s_t = decay^(p_t) * (sum over the request's tokens j <= t of this step of decay^(-p_j) x_j
                         + decay^(1 - first) * s_before), with s_before = 0 for a request that starts at 0
    (p: absolute positions; first: the position of the request's first token in this step)."""

    recordable = True

    def forward(self, x, step, cache):
        pool = cache.state["sum"]
        batch = step.attention
        req = batch.token_req.long()
        pos = batch.positions.to(torch.float64)                         # the tokens' indices in their requests
        first_row = batch.cu_seqlens_q[:-1].long()                      # [B] row of every request's first token
        last_row = batch.cu_seqlens_q[1:].long() - 1
        slots = step.state_slots.long()
        log_decay = math.log(self.decay)

        def power(exponent):                                            # decay^exponent, from device tensors only
            return torch.exp(exponent * log_decay)

        y = x.to(torch.float64) * power(-pos)[:, None]
        c = torch.cumsum(y, dim=0)
        within = c - (c[first_row] - y[first_row])[req]                # sums that start at the request's first row
        first_pos = pos[first_row]
        before = torch.where((first_pos == 0)[:, None], torch.zeros_like(pool[slots], dtype=torch.float64),
                             pool[slots].to(torch.float64))
        carried = before * power(1.0 - first_pos)[:, None]
        s = (within + carried[req]) * power(pos)[:, None]
        pool[slots] = s[last_row].to(pool.dtype)
        return (s.to(torch.float32) @ self.weight.float().T).to(x.dtype)


class RoutedFeedForward(Part):
    """Toy feed-forward with routing: router logits and their softmax in float32; every token goes through
    the expert it rates highest (the experts are the package's own gated feed-forwards, built through the
    registry) and the result is weighted with that expert's probability."""

    def __init__(self, hidden_size: int, intermediate_size: int, num_experts: int, on_device: bool = False):
        self.hidden_size = hidden_size
        # False: the rows of every expert are looked up on the host and only those go through it (a step with
        # this cannot be recorded); True: every expert sees every row and a mask keeps the chosen ones
        self.recordable = on_device
        self.experts = [FEED_FORWARDS.build({"kind": "swiglu", "hidden_size": hidden_size,
                                             "intermediate_size": intermediate_size}) for _ in range(num_experts)]

    def param_specs(self):
        return {"router.weight": ParamSpec((len(self.experts), self.hidden_size), keeps_float32=True)}

    def children(self):
        return {f"experts.{i}": e for i, e in enumerate(self.experts)}

    def bind(self, params):
        self.router = params["router.weight"]

    def forward(self, x, step):
        prob = torch.softmax(x.float() @ self.router.float().T, dim=-1)
        best = prob.argmax(dim=-1)
        out = torch.zeros_like(x)
        if self.recordable:
            for e, expert in enumerate(self.experts):
                y = expert.forward(x, step).float() * prob[:, e:e + 1]
                out = torch.where((best == e)[:, None], y.to(x.dtype), out)
            return out
        for e, expert in enumerate(self.experts):
            rows = (best == e).nonzero().flatten()
            if rows.numel():
                y = expert.forward(x[rows].contiguous(), step)
                out[rows] = (y.float() * prob[rows, e:e + 1]).to(x.dtype)
        return out


class LinearAngles(Part):
    """Toy position encoding: the angle of pair j at position p is p * (j + 1) * step, only the first
    ``rotary_dim`` entries of a head are turned, and p is the coordinate of axis j % axes of the token's position."""

    def __init__(self, rotary_dim: int, step: float, max_position: int, axes: int = 1, device=None):
        ang = torch.arange(max_position, dtype=torch.float32)[:, None] * (torch.arange(rotary_dim // 2) + 1.0) * step
        self.table = torch.cat((ang.cos(), ang.sin()), dim=-1).contiguous()
        self.axes = (torch.arange(rotary_dim // 2) % axes).to(torch.int32) if axes > 1 else None

    def rotation_table(self):
        return self.table

    def pair_axes(self):
        return self.axes

    def to(self, device):
        self.table = self.table.to(device)
        if self.axes is not None:
            self.axes = self.axes.to(device)
        return self


class SandwichBlock(Part):
    """Toy block arrangement with three norms: r += post_mixer_norm(mixer(mixer_norm(r))); r += feed_forward(
    feed_forward_norm(r)). It keeps the engine's convention of (hidden, residual) with the second addition left to
    the next norm."""

    norm_slots = ("mixer_norm", "post_mixer_norm", "feed_forward_norm")

    def __init__(self, mixer, feed_forward, mixer_norm, post_mixer_norm, feed_forward_norm):
        self.mixer, self.feed_forward = mixer, feed_forward
        self.mixer_norm, self.post_mixer_norm, self.feed_forward_norm = mixer_norm, post_mixer_norm, feed_forward_norm

    def children(self):
        return {"mixer_norm": self.mixer_norm, "mixer": self.mixer, "post_mixer_norm": self.post_mixer_norm,
                "feed_forward_norm": self.feed_forward_norm, "feed_forward": self.feed_forward}

    def forward(self, hidden, residual, step, cache):
        if residual is None:
            x, residual = self.mixer_norm.forward_start(hidden)
        else:
            x, residual = self.mixer_norm.forward_add(hidden, residual)
        x = self.post_mixer_norm.forward(self.mixer.forward(x, step, cache))
        x, residual = self.feed_forward_norm.forward_add(x, residual)
        return self.feed_forward.forward(x, step), residual


def toy_spec(cfg: dict) -> ModelSpec:
    state_mixer = "toy_decaying_sum_on_device" if cfg.get("device_state") else "toy_decaying_sum"
    norm = {"kind": "rmsnorm", "size": H, "eps": 1e-5}
    ff = {"kind": "swiglu", "hidden_size": H, "intermediate_size": INTER}

    def attention(window):
        return {"kind": "gqa_attention", "hidden_size": H, "num_heads": HEADS, "num_kv_heads": KV, "head_dim": D,
                "scale": D ** -0.5, "qk_norm_eps": 1e-5, "qkv_bias": False, "window": window}
    routed = {"kind": "toy_routed", "hidden_size": H, "intermediate_size": EXPERT_INTER, "num_experts": EXPERTS,
              "on_device": bool(cfg.get("device_state"))}
    layers = [
        LayerSpec(mixer=attention(None), feed_forward=ff, norm=norm, block={"kind": "toy_sandwich"},
                  norms={"post_mixer_norm": {"kind": "rmsnorm", "size": H, "eps": POST_EPS}}),
        LayerSpec(mixer={"kind": state_mixer, "hidden_size": H, "decay": DECAY}, feed_forward=routed, norm=norm),
        LayerSpec(mixer=attention(None if cfg.get("no_window") else WINDOW), feed_forward=ff, norm=norm, position="linear"),
    ]
    # layer 0 runs twice (two caches); the last entry runs layer 2 again on the keys and values of entry 2
    order = [RunEntry(0), RunEntry(1), RunEntry(2), RunEntry(0), RunEntry(2, cache=2)]
    return ModelSpec(vocab_size=VOCAB, hidden_size=H, layers=layers, final_norm=norm,
                     positions={"default": {"kind": "rope", "rotary_dim": D, "base": 1000.0},
                                "linear": {"kind": "toy_linear_angles", "rotary_dim": TOY_ROT, "step": TOY_STEP, "axes": AXES}},
                     max_position=256, tie_embeddings=True, run_order=order, eos_token_id=cfg.get("eos_token_id"),
                     embed_scale=EMBED_SCALE, logit_cap=LOGIT_CAP, position_axes=AXES)


def toy_names(cfg):
    return {name: WeightSource(name) for name in DecoderModel(toy_spec(cfg)).all_param_specs()}


def toy_turn(x, pos):
    """The toy position encoding on [T, heads, D]: pairs (j, j + TOY_ROT / 2) of the first TOY_ROT entries; pair j
    turns by the coordinate of axis j % AXES (``pos``: [AXES, T])."""
    j = torch.arange(TOY_ROT // 2)
    ang = pos.float()[j % AXES].T * (j + 1.0) * TOY_STEP
    cos, sin = ang.cos()[:, None, :], ang.sin()[:, None, :]
    x1, x2 = x[..., :TOY_ROT // 2], x[..., TOY_ROT // 2:TOY_ROT]
    return torch.cat((x1 * cos - x2 * sin, x2 * cos + x1 * sin, x[..., TOY_ROT:]), dim=-1)


def toy_plain_logits(w, toks, no_window=False, positions=None):
    """Whole sequence, no cache, from the plain functions. ``positions``: [AXES, T] coordinates for the encoding
    over several axes (default: the tokens' indices on every axis)."""
    window_of_layer_2 = None if no_window else WINDOW
    T = len(toks)
    pos = torch.arange(T)
    axes_pos = torch.stack([pos] * AXES) if positions is None else torch.as_tensor(positions)
    r = w["embed.weight"][toks] * EMBED_SCALE
    kept = {}

    def attention(x, p, window, entry, lender=None):
        # layer 2 has the toy angles over both axes; the other layers' rotation takes the first axis, the index
        turn = (lambda t, at: toy_turn(t, axes_pos)) if p.startswith("layers.2.") else (lambda t, at: plain.apply_rope(t, at, 1000.0))
        qkv = x @ w[p + "mixer.qkv.weight"].T
        q = plain.rms_norm(qkv[:, :HEADS * D].view(T, HEADS, D), w[p + "mixer.q_norm.weight"], 1e-5)
        if lender is None:
            k = plain.rms_norm(qkv[:, HEADS * D:(HEADS + KV) * D].view(T, KV, D), w[p + "mixer.k_norm.weight"], 1e-5)
            v = qkv[:, (HEADS + KV) * D:].view(T, KV, D)
            kept[entry] = (turn(k, pos), v)
        k, v = kept[entry if lender is None else lender]
        o = plain.causal_attention(turn(q, pos), k, v, D ** -0.5, window)
        return o.reshape(T, HEADS * D) @ w[p + "mixer.o.weight"].T

    def routed(x, p):
        prob = torch.softmax(x @ w[p + "feed_forward.router.weight"].T, dim=-1)
        rows = []
        for t in range(T):
            e = int(prob[t].argmax())
            gu = w[p + f"feed_forward.experts.{e}.gate_up.weight"]
            y = plain.swiglu(x[t:t + 1], gu[:EXPERT_INTER], gu[EXPERT_INTER:], w[p + f"feed_forward.experts.{e}.down.weight"])
            rows.append(y[0] * prob[t, e])
        return torch.stack(rows)

    def decaying_sum(x, p):
        s, rows = torch.zeros(H), []
        for t in range(T):
            s = DECAY * s + x[t]
            rows.append(s @ w[p + "mixer.out.weight"].T)
        return torch.stack(rows)

    for entry, (layer, lender) in enumerate([(0, None), (1, None), (2, None), (0, None), (2, 2)]):
        p = f"layers.{layer}."
        x = plain.rms_norm(r, w[p + "mixer_norm.weight"], 1e-5)
        if layer == 1:
            r = r + decaying_sum(x, p)
        elif layer == 0:                     # the sandwich block: a norm of its own after the mixer
            r = r + plain.rms_norm(attention(x, p, None, entry, lender), w[p + "post_mixer_norm.weight"], POST_EPS)
        else:
            r = r + attention(x, p, window_of_layer_2, entry, lender)
        x = plain.rms_norm(r, w[p + "feed_forward_norm.weight"], 1e-5)
        if layer == 1:
            r = r + routed(x, p)
            continue
        gu = w[p + "feed_forward.gate_up.weight"]
        r = r + plain.swiglu(x, gu[:INTER], gu[INTER:], w[p + "feed_forward.down.weight"])
    logits = plain.rms_norm(r, w["final_norm.weight"], 1e-5) @ w["embed.weight"].T
    return LOGIT_CAP * torch.tanh(logits / LOGIT_CAP)


_PARTS = [(MIXERS, "toy_decaying_sum", DecayingSum), (MIXERS, "toy_decaying_sum_on_device", DecayingSumOnDevice),
          (FEED_FORWARDS, "toy_routed", RoutedFeedForward), (POSITION_ENCODINGS, "toy_linear_angles", LinearAngles),
          (BLOCKS, "toy_sandwich", SandwichBlock)]


def register_parts() -> None:
    for registry, kind, maker in _PARTS:
        if kind not in registry.kinds():
            registry.register(kind)(maker)


def unregister_parts() -> None:
    for registry, kind, _ in _PARTS:
        registry.unregister(kind)


def register() -> None:
    register_parts()
    register_architecture(Architecture("ToyForCausalLM", ("toy",), dict, toy_spec, toy_names), replace=True)


def unregister() -> None:
    unregister_architecture("ToyForCausalLM")
    unregister_parts()


register()

"""The parts are general: a toy architecture, defined here and nowhere in the package,
with a mixer that keeps state of its own per request, a feed-forward that routes every
token to one of several experts, a position encoding of its own (other angles, on a
part of the head only), a layer with a window (pages of its own, given back as the
window passes), a layer that runs twice and an entry that reads another entry's cache,
is registered, built, loaded and stepped through the unchanged engine and compared
with a plain whole-sequence computation.
Also: each built-in part alone against its plain function."""
import pytest
import torch

import plain_qwen3 as plain
import replay_cases as rc
from helpers import max_abs_diff
from nanohybrid_vlm_amd.cache.manager import NO_PAGE
from nanohybrid_vlm_amd.config.registry import (Architecture, WeightSource, register_architecture,
                                                unregister_architecture)
from nanohybrid_vlm_amd.parts import FEED_FORWARDS, MIXERS, POSITION_ENCODINGS, ParamSpec, Part, StateNeed
from nanohybrid_vlm_amd.parts.model import DecoderModel, LayerSpec, ModelSpec, RunEntry
from nanohybrid_vlm_amd.weights.random_init import write_random_model

H, HEADS, KV, D, INTER, VOCAB, WINDOW, DECAY = 48, 3, 1, 16, 64, 97, 5, 0.75
EXPERTS, EXPERT_INTER, TOY_ROT, TOY_STEP = 3, 40, 8, 0.05


class DecayingSum(Part):
    """Toy mixer with state: s_t = decay * s_(t-1) + x_t per request, output s_t W^T.
    The state of a request lives in its state slot between steps."""

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


class RoutedFeedForward(Part):
    """Toy feed-forward with routing: router logits and their softmax in float32; every token goes through
    the expert it rates highest (the experts are the package's own gated feed-forwards, built through the
    registry) and the result is weighted with that expert's probability."""

    def __init__(self, hidden_size: int, intermediate_size: int, num_experts: int):
        self.hidden_size = hidden_size
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
        for e, expert in enumerate(self.experts):
            rows = (best == e).nonzero().flatten()
            if rows.numel():
                y = expert.forward(x[rows].contiguous(), step)
                out[rows] = (y.float() * prob[rows, e:e + 1]).to(x.dtype)
        return out


class LinearAngles(Part):
    """Toy position encoding: the angle of pair j at position p is p * (j + 1) * step, and only the first
    ``rotary_dim`` entries of a head are turned."""

    def __init__(self, rotary_dim: int, step: float, max_position: int, device=None):
        ang = torch.arange(max_position, dtype=torch.float32)[:, None] * (torch.arange(rotary_dim // 2) + 1.0) * step
        self.table = torch.cat((ang.cos(), ang.sin()), dim=-1).contiguous()

    def rotation_table(self):
        return self.table

    def to(self, device):
        self.table = self.table.to(device)
        return self


def toy_spec(cfg: dict) -> ModelSpec:
    norm = {"kind": "rmsnorm", "size": H, "eps": 1e-5}
    ff = {"kind": "swiglu", "hidden_size": H, "intermediate_size": INTER}

    def attention(window):
        return {"kind": "gqa_attention", "hidden_size": H, "num_heads": HEADS, "num_kv_heads": KV, "head_dim": D,
                "scale": D ** -0.5, "qk_norm_eps": 1e-5, "qkv_bias": False, "window": window}
    routed = {"kind": "toy_routed", "hidden_size": H, "intermediate_size": EXPERT_INTER, "num_experts": EXPERTS}
    layers = [
        LayerSpec(mixer=attention(None), feed_forward=ff, norm=norm),
        LayerSpec(mixer={"kind": "toy_decaying_sum", "hidden_size": H, "decay": DECAY}, feed_forward=routed, norm=norm),
        LayerSpec(mixer=attention(WINDOW), feed_forward=ff, norm=norm, position="linear"),
    ]
    # layer 0 runs twice (two caches); the last entry runs layer 2 again on the keys and values of entry 2
    order = [RunEntry(0), RunEntry(1), RunEntry(2), RunEntry(0), RunEntry(2, cache=2)]
    return ModelSpec(vocab_size=VOCAB, hidden_size=H, layers=layers, final_norm=norm,
                     positions={"default": {"kind": "rope", "rotary_dim": D, "base": 1000.0},
                                "linear": {"kind": "toy_linear_angles", "rotary_dim": TOY_ROT, "step": TOY_STEP}},
                     max_position=256, tie_embeddings=True, run_order=order)


def toy_names(cfg):
    return {name: WeightSource(name) for name in DecoderModel(toy_spec(cfg)).all_param_specs()}


@pytest.fixture()
def toy_architecture():
    _register_toy_parts()
    register_architecture(Architecture("ToyForCausalLM", ("toy",), dict, toy_spec, toy_names))
    yield
    unregister_architecture("ToyForCausalLM")
    _unregister_toy_parts()


def _register_toy_parts():
    MIXERS.register("toy_decaying_sum")(DecayingSum)
    FEED_FORWARDS.register("toy_routed")(RoutedFeedForward)
    POSITION_ENCODINGS.register("toy_linear_angles")(LinearAngles)


def _unregister_toy_parts():
    MIXERS.unregister("toy_decaying_sum")
    FEED_FORWARDS.unregister("toy_routed")
    POSITION_ENCODINGS.unregister("toy_linear_angles")


def toy_turn(x, pos):
    """The toy position encoding on [T, heads, D]: pairs (j, j + TOY_ROT / 2) of the first TOY_ROT entries."""
    ang = pos.float()[:, None] * (torch.arange(TOY_ROT // 2) + 1.0) * TOY_STEP
    cos, sin = ang.cos()[:, None, :], ang.sin()[:, None, :]
    x1, x2 = x[..., :TOY_ROT // 2], x[..., TOY_ROT // 2:TOY_ROT]
    return torch.cat((x1 * cos - x2 * sin, x2 * cos + x1 * sin, x[..., TOY_ROT:]), dim=-1)


def toy_plain_logits(w, toks):
    """Whole sequence, no cache, from the plain functions."""
    T = len(toks)
    pos = torch.arange(T)
    r = w["embed.weight"][toks]
    kept = {}

    def attention(x, p, window, entry, lender=None):
        turn = toy_turn if window else (lambda t, at: plain.apply_rope(t, at, 1000.0))   # the windowed layer has the toy angles
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
        else:
            r = r + attention(x, p, WINDOW if layer == 2 else None, entry, lender)
        x = plain.rms_norm(r, w[p + "feed_forward_norm.weight"], 1e-5)
        if layer == 1:
            r = r + routed(x, p)
            continue
        gu = w[p + "feed_forward.gate_up.weight"]
        r = r + plain.swiglu(x, gu[:INTER], gu[INTER:], w[p + "feed_forward.down.weight"])
    return plain.rms_norm(r, w["final_norm.weight"], 1e-5) @ w["embed.weight"].T


def _toy_check(device, dtype, tol, tmp_path):
    from nanohybrid_vlm_amd.engine.runner import ModelRunner
    cfg = {"architectures": ["ToyForCausalLM"], "model_type": "toy"}
    folder = write_random_model(str(tmp_path / "toy"), cfg, seed=4)
    _, w = plain.read_model_folder(folder)
    requests = {f"r{i}": rc.random_tokens(VOCAB, n, 30 + i) for i, n in enumerate([9, 40, 23, 17, 31])}
    want = {rid: toy_plain_logits(w, toks) for rid, toks in requests.items()}
    for mode, steps in [("whole", rc.whole(requests)), ("portions", rc.portions(requests)),
                        ("mixed", rc.mixed(requests, max_live=3))]:
        pages = rc.peak_tokens(steps, 4) // 4
        runner = ModelRunner(folder, dtype=dtype, device=device, page_size=4, num_pages=pages, num_state_slots=3)
        assert len(runner.cache.groups) == 2 and runner.cache.groups[1].window == WINDOW
        assert len(runner.kv_tensors) == 3 and len(runner.state_pools) == 1       # entries 0, 2, 3 store keys; entry 1 state
        got = rc.run_in_process(runner, steps)
        for rid in requests:
            d = max_abs_diff(got[rid], want[rid])
            assert d <= tol, f"toy {mode}: request {rid}: {d:.3e}"
        assert all(runner.cache.num_free_pages(g) == pages for g in range(2))
    # the windowed group gives pages back while a request is still alive
    runner = ModelRunner(folder, dtype=dtype, device=device, page_size=4, num_pages=16, num_state_slots=3)
    from nanohybrid_vlm_amd.engine.runner import StepEntry
    runner.step([StepEntry("x", requests["r1"][:30], [29])])
    assert runner.cache.block_table("x", 0).count(NO_PAGE) == 0
    assert runner.cache.block_table("x", 1).count(NO_PAGE) == (30 - WINDOW + 1) // 4


def test_toy_architecture_on_emulated_kernels(toy_architecture, emulated_kernels, tmp_path):
    _toy_check("cpu", "float32", 2e-5, tmp_path)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,tol", [("float32", 2e-5), ("bfloat16", 3e-2)])
def test_toy_architecture_on_gpu(toy_architecture, dtype, tol, tmp_path):
    _toy_check("cuda:0", dtype, tol, tmp_path)


def test_run_order_is_checked():
    spec = toy_spec({})
    _register_toy_parts()
    try:
        spec.run_order = [RunEntry(0), RunEntry(5)]
        with pytest.raises(ValueError, match="names layer 5"):
            DecoderModel(spec)
        spec.run_order = [RunEntry(0), RunEntry(2, cache=0)]                      # a window layer on an all-keys cache
        with pytest.raises(ValueError, match="different caches"):
            DecoderModel(spec)
        spec.run_order = [RunEntry(0, cache=0)]
        with pytest.raises(ValueError, match="earlier entry"):
            DecoderModel(spec)
    finally:
        _unregister_toy_parts()
    with pytest.raises(KeyError, match="unknown position encoding"):
        DecoderModel(toy_spec({}))


# ---------------------------------------------------------------- built-in parts alone, on the GPU
def _dev(t, dtype):
    return t.to(dtype).cuda()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_builtin_parts_alone(dtype):
    from nanohybrid_vlm_amd.parts.feed_forward import SwiGLU
    from nanohybrid_vlm_amd.parts.norms import RMSNorm
    from nanohybrid_vlm_amd.parts.positions import RotaryEmbedding
    tol = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    g = torch.Generator().manual_seed(0)
    x = torch.randn(11, 72, generator=g).to(dtype)
    # norm
    norm = RMSNorm(72, 1e-4)
    wn = (1 + 0.1 * torch.randn(72, generator=g)).to(dtype)
    norm.bind({"weight": wn.cuda()})
    torch.testing.assert_close(norm.forward(x.cuda()).float().cpu(), plain.rms_norm(x, wn.float(), 1e-4), **tol)
    y, res = norm.forward_start(x.cuda())
    y2, res = norm.forward_add(x.cuda(), res)
    ref, s = plain.add_rms_norm(x, x, wn.float(), 1e-4)
    torch.testing.assert_close(y2.float().cpu(), ref, **tol)
    assert torch.equal(res.cpu(), s)
    # feed-forward
    ff = SwiGLU(72, 100)
    gu = (torch.randn(200, 72, generator=g) * 0.1).to(dtype)
    dn = (torch.randn(72, 100, generator=g) * 0.1).to(dtype)
    ff.bind({"gate_up.weight": gu.cuda(), "down.weight": dn.cuda()})
    assert set(ff.param_specs()) == {"gate_up.weight", "down.weight"}
    torch.testing.assert_close(ff.forward(x.cuda(), None).float().cpu(),
                               plain.swiglu(x.float(), gu[:100].float(), gu[100:].float(), dn.float()), **tol)
    # position encoding: its table holds the plain angles
    rope = RotaryEmbedding(rotary_dim=24, max_position=50, base=500.0)
    ang = plain.rope_angles(torch.arange(50), 24, 500.0)
    torch.testing.assert_close(rope.rotation_table(), torch.cat((ang.cos(), ang.sin()), -1))

"""Pins of the plain implementation beside the reference's text: special cases that
reduce to a library routine and invariants, each chosen so that a plausible mistake
(a wrong sign or pairing, a swapped gate, a norm in the wrong place, a wrong group
mapping) fails it. The reference holds no test vector for Qwen3 dense (its golden
files are of another architecture), so whole-model parity is unpinned beyond these."""
import math

import pytest
import torch
import torch.nn.functional as F

import plain_qwen3 as plain
from conftest import TINY_A, TINY_B


def test_rms_norm_is_the_library_routine():
    x = torch.randn(5, 96) * 3
    w = 1 + 0.1 * torch.randn(96)
    torch.testing.assert_close(plain.rms_norm(x, w, 1e-5), F.rms_norm(x, (96,), w, 1e-5))
    # eps sits inside the root, added to the mean of squares: ||y||^2 = H ||x||^2 / (||x||^2 + H eps) for w = 1
    eps = 0.5
    y = plain.rms_norm(x, torch.ones(96), eps)
    n2 = x.pow(2).sum(-1)
    torch.testing.assert_close(y.pow(2).sum(-1), 96 * n2 / (n2 + 96 * eps))


def test_add_rms_norm_norms_the_sum_and_carries_it():
    x, r = torch.randn(4, 32), torch.randn(4, 32)
    w = 1 + 0.1 * torch.randn(32)
    y, s = plain.add_rms_norm(x, r, w, 1e-6)
    assert torch.equal(s, x + r)
    torch.testing.assert_close(y, plain.rms_norm(x + r, w, 1e-6))


def test_rope_angles_against_float64():
    pos = torch.arange(0, 300, 7)
    for base, d in [(10000.0, 16), (1e6, 32), (50000.0, 48)]:
        ang = plain.rope_angles(pos, d, base).double()
        ref = pos.double()[:, None] * torch.tensor([base ** (-2 * j / d) for j in range(d // 2)], dtype=torch.float64)
        torch.testing.assert_close(ang, ref, rtol=2e-6, atol=1e-4)


def test_rope_pairs_first_half_with_second_half():
    d = 16
    x = torch.zeros(1, 1, d)
    x[0, 0, 0] = 1.0                                       # only the first entry of the first half
    y = plain.apply_rope(x, torch.tensor([3]), 10000.0)[0, 0]
    # pair (0, d/2) turns by 3 * base^0 = 3 rad: (1, 0) -> (cos 3, sin 3); an interleaved pairing would fill y[1]
    assert abs(y[0] - math.cos(3.0)) < 1e-6 and abs(y[d // 2] - math.sin(3.0)) < 1e-6
    assert y[1] == 0 and y[d // 2 + 1] == 0
    # the last pair turns slowest
    x = torch.zeros(1, 1, d)
    x[0, 0, d // 2 - 1] = 1.0
    y = plain.apply_rope(x, torch.tensor([3]), 10000.0)[0, 0]
    a = 3 * 10000.0 ** (-(d - 2) / d)
    assert abs(y[d // 2 - 1] - math.cos(a)) < 1e-6 and abs(y[d - 1] - math.sin(a)) < 1e-6


def test_rope_invariants():
    q, k = torch.randn(9, 3, 32), torch.randn(9, 3, 32)
    pos = torch.arange(9)
    # position 0 is the identity
    torch.testing.assert_close(plain.apply_rope(q[:1], pos[:1], 1e6), q[:1])
    # lengths of pairs are kept
    y = plain.apply_rope(q, pos + 11, 1e6)
    torch.testing.assert_close(y[..., :16] ** 2 + y[..., 16:] ** 2, q[..., :16] ** 2 + q[..., 16:] ** 2)
    # a product of a turned q and a turned k depends on the distance only
    a = (plain.apply_rope(q, pos + 5, 1e4) * plain.apply_rope(k, pos + 2, 1e4)).sum(-1)
    b = (plain.apply_rope(q, pos + 105, 1e4) * plain.apply_rope(k, pos + 102, 1e4)).sum(-1)
    torch.testing.assert_close(a, b, rtol=1e-4, atol=1e-4)
    # and with the sign of the sine flipped it would not equal the complex product
    z = torch.complex(q[..., :16], q[..., 16:]) * torch.polar(torch.ones(9, 1, 16), plain.rope_angles(pos + 11, 32, 1e6)[:, None, :])
    torch.testing.assert_close(y, torch.cat((z.real, z.imag), -1))


def test_attention_is_the_library_routine_for_full_heads():
    T, H, D = 23, 4, 16
    q, k, v = torch.randn(T, H, D), torch.randn(T, H, D), torch.randn(T, H, D)
    ref = F.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1), is_causal=True,
                                         scale=D ** -0.5).transpose(0, 1)
    torch.testing.assert_close(plain.causal_attention(q, k, v, D ** -0.5), ref, rtol=1e-5, atol=1e-5)


def test_attention_groups_and_special_cases():
    T, Hq, Hkv, D = 11, 6, 2, 8
    q, k, v = torch.randn(T, Hq, D), torch.randn(T, Hkv, D), torch.randn(T, Hkv, D)
    out = plain.causal_attention(q, k, v, 0.3)
    # grouped heads equal full heads after repeating each kv head Hq/Hkv times in place (head h reads h // 3)
    full = plain.causal_attention(q, k.repeat_interleave(3, dim=1), v.repeat_interleave(3, dim=1), 0.3)
    torch.testing.assert_close(out, full)
    assert not torch.allclose(out, plain.causal_attention(q, k.repeat(1, 3, 1), v.repeat(1, 3, 1), 0.3))
    # the first position sees one key: its output is that value
    torch.testing.assert_close(out[0], v[0].repeat_interleave(3, dim=0))
    # a window of one sees only itself
    torch.testing.assert_close(plain.causal_attention(q, k, v, 0.3, window=1), v.repeat_interleave(3, dim=1))
    # a window as long as the sequence changes nothing
    torch.testing.assert_close(plain.causal_attention(q, k, v, 0.3, window=T), out)


def test_swiglu_gate_is_the_first_matrix():
    x = torch.randn(5, 12)
    wg, wu, wd = torch.randn(20, 12), torch.randn(20, 12), torch.randn(12, 20)
    torch.testing.assert_close(plain.swiglu(x, wg, wu, wd), (F.silu(x @ wg.T) * (x @ wu.T)) @ wd.T)
    assert not torch.allclose(plain.swiglu(x, wg, wu, wd), plain.swiglu(x, wu, wg, wd))


def _random_weights(cfg, seed):
    from nanohybrid_vlm_amd.weights.random_init import random_checkpoint_tensors
    return {k: v.float() for k, v in random_checkpoint_tensors(cfg, seed).items()}


@pytest.mark.parametrize("cfg,seed", [(TINY_A, 0), (TINY_B, 1)])
def test_only_distances_between_positions_count(cfg, seed):
    """Shifting all positions leaves the logits alone: positions enter through the rotation only."""
    w = _random_weights(cfg, seed)
    toks = torch.randint(0, cfg["vocab_size"], (19,)).tolist()
    a = plain.logits(cfg, w, toks, first_position=0)
    b = plain.logits(cfg, w, toks, first_position=37)
    torch.testing.assert_close(a, b, rtol=1e-4, atol=2e-5)


@pytest.mark.parametrize("cfg,seed", [(TINY_A, 0), (TINY_B, 1)])
def test_stored_results_rounded_to_bfloat16(cfg, seed):
    """``stored_as(bfloat16)`` rounds where the reference's bfloat16 model stores (nanovllm/layers/layernorm.py:25,
    rotary_embedding.py:13): the parts' results are then bfloat16 numbers, a norm rounds the scaled row before the
    weight, the logits move by some bfloat16 roundings and no more, and leaving the block restores float32."""
    w = _random_weights(cfg, seed)
    toks = torch.randint(0, cfg["vocab_size"], (23,)).tolist()
    exact = plain.logits(cfg, w, toks)
    x = torch.randn(7, 24)
    weight = 1 + 0.1 * torch.randn(24)
    with plain.stored_as(torch.bfloat16):
        rounded = plain.logits(cfg, w, toks)
        y = plain.rms_norm(x, weight, 1e-6)
        r = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6)
        assert torch.equal(y, (r.bfloat16().float() * weight).bfloat16().float())
        assert not torch.equal(y, (r * weight).bfloat16().float())          # (rounding once would differ somewhere)
        h = plain.hidden_states(cfg, w, toks)
        assert torch.equal(h, h.bfloat16().float())
    assert torch.equal(plain.logits(cfg, w, toks), exact)
    diff = (rounded - exact).abs().max().item()
    assert 1e-4 < diff < 0.05 * exact.abs().max().item(), diff


def test_causality_and_dead_layers():
    cfg = TINY_A
    w = _random_weights(cfg, 0)
    toks = torch.randint(0, cfg["vocab_size"], (15,)).tolist()
    full = plain.logits(cfg, w, toks)
    # a position does not see later tokens
    torch.testing.assert_close(plain.logits(cfg, w, toks[:9]), full[:9], rtol=1e-5, atol=1e-6)
    # with the output projections of every layer at zero the layers add nothing:
    # logits = norm(embedding) . embedding^T (tied), which fixes where the final norm sits
    dead = dict(w)
    for name in w:
        if name.endswith("o_proj.weight") or name.endswith("down_proj.weight"):
            dead[name] = torch.zeros_like(w[name])
    e = w["model.embed_tokens.weight"]
    ref = F.rms_norm(e[toks], (cfg["hidden_size"],), w["model.norm.weight"], cfg["rms_norm_eps"]) @ e.T
    torch.testing.assert_close(plain.logits(cfg, dead, toks), ref, rtol=1e-5, atol=1e-6)


def test_one_layer_one_head_by_hand():
    """One layer, one head, one kv head: every step spelled out with library calls."""
    cfg = dict(TINY_A, num_hidden_layers=1, num_attention_heads=1, num_key_value_heads=1, head_dim=16, hidden_size=16,
               intermediate_size=24, vocab_size=50, tie_word_embeddings=False)
    w = _random_weights(cfg, 3)
    toks = [4, 9, 1, 30, 7]
    eps = cfg["rms_norm_eps"]
    p = "model.layers.0."
    r = w["model.embed_tokens.weight"][toks]
    x = F.rms_norm(r, (16,), w[p + "input_layernorm.weight"], eps)
    q = F.rms_norm(x @ w[p + "self_attn.q_proj.weight"].T, (16,), w[p + "self_attn.q_norm.weight"], eps)
    k = F.rms_norm(x @ w[p + "self_attn.k_proj.weight"].T, (16,), w[p + "self_attn.k_norm.weight"], eps)
    v = x @ w[p + "self_attn.v_proj.weight"].T
    pos = torch.arange(5)
    ang = pos[:, None].float() * (10000.0 ** (-torch.arange(0, 16, 2).float() / 16))[None]
    rot = lambda t: torch.cat((t[:, :8] * ang.cos() - t[:, 8:] * ang.sin(), t[:, 8:] * ang.cos() + t[:, :8] * ang.sin()), -1)
    o = F.scaled_dot_product_attention(rot(q)[None], rot(k)[None], v[None], is_causal=True, scale=0.25)[0]
    r = r + o @ w[p + "self_attn.o_proj.weight"].T
    x = F.rms_norm(r, (16,), w[p + "post_attention_layernorm.weight"], eps)
    r = r + (F.silu(x @ w[p + "mlp.gate_proj.weight"].T) * (x @ w[p + "mlp.up_proj.weight"].T)) @ w[p + "mlp.down_proj.weight"].T
    ref = F.rms_norm(r, (16,), w["model.norm.weight"], eps) @ w["lm_head.weight"].T
    torch.testing.assert_close(plain.logits(cfg, w, toks), ref, rtol=1e-5, atol=1e-6)


def test_sampling_rule():
    row = torch.tensor([0.1, 2.0, 2.0, -1.0])
    assert plain.sample_token(row, 0.0, None) == 1                      # argmax, first of equals
    noise = torch.tensor([1e-3, 1.0, 1.0, 1.0])                          # tiny noise on index 0 wins: p / noise
    assert plain.sample_token(row, 1.0, noise) == 0
    n = plain.sample_noise(5, 2, 3, 1000)
    assert (n >= 0).all() and abs(n.mean().item() - 1.0) < 0.1            # Exp(1) has mean 1
    assert torch.equal(n, plain.sample_noise(5, 2, 3, 1000))
    assert not torch.equal(n, plain.sample_noise(5, 2, 4, 1000))


def test_noise_of_the_extreme_bit_patterns():
    """The 24 bits' noise is the middle of their bucket of the Exp(1) distribution: the lowest noise is 3e-8, which
    is what a true draw below 6e-8 is on average, and not 0 (or a floor of 1e-10, which would let an index of
    chance 1e-9 win once in 2^24 draws); the share of patterns below x is 1 - exp(-x) to within one pattern."""
    import math
    import numpy as np
    n = 1 << 24
    assert math.isclose(plain.noise_of_bits(n - 1), 0.5 / n, rel_tol=1e-6)
    assert math.isclose(plain.noise_of_bits(0), math.log(2 * n), rel_tol=1e-12)
    values = np.array([plain.noise_of_bits(b) for b in list(range(n - 2000, n)) + list(range(0, n, 4099))])
    assert (values > 2.9e-8).all() and np.isfinite(values).all()
    for x in (1e-7, 1e-6, 1e-5, 1e-3, 0.5):
        below = sum(1 for b in range(n - 1, n - 200, -1) if plain.noise_of_bits(b) < x) if x < 1e-5 else None
        if below is not None:
            assert abs(below / n - (1 - math.exp(-x))) <= 1.0 / n


# ---------------------------------------------------------------- readings that no library routine fixes
def _variant_logits(cfg, w, toks, first_position=0, norm_after_rotation=False, post_norm=False, scale_power=-0.5):
    """The model from the plain part functions with three switches, each a plausible misreading of the reference:
    the per-head norms of q and k after the rotation instead of before it (nanovllm/models/qwen3.py:82-85), a
    post-norm block instead of the pre-norm one with the addition carried on (qwen3.py:152-159), and another power
    of the head size as the scale (qwen3.py:39). With all switches off it is the plain implementation."""
    Hq, Hkv, D = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    eps, theta = cfg["rms_norm_eps"], cfg["rope_theta"]
    T = len(toks)
    pos = torch.arange(first_position, first_position + T)
    r = w["model.embed_tokens.weight"][toks]
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."

        def attention(x):
            q = (x @ w[p + "self_attn.q_proj.weight"].T).view(T, Hq, D)
            k = (x @ w[p + "self_attn.k_proj.weight"].T).view(T, Hkv, D)
            v = (x @ w[p + "self_attn.v_proj.weight"].T).view(T, Hkv, D)
            qn, kn = w[p + "self_attn.q_norm.weight"], w[p + "self_attn.k_norm.weight"]
            if norm_after_rotation:
                q = plain.rms_norm(plain.apply_rope(q, pos, theta), qn, eps)
                k = plain.rms_norm(plain.apply_rope(k, pos, theta), kn, eps)
            else:
                q = plain.apply_rope(plain.rms_norm(q, qn, eps), pos, theta)
                k = plain.apply_rope(plain.rms_norm(k, kn, eps), pos, theta)
            return plain.causal_attention(q, k, v, D ** scale_power).reshape(T, Hq * D) @ w[p + "self_attn.o_proj.weight"].T

        def feed_forward(x):
            return plain.swiglu(x, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])

        if post_norm:
            r = plain.rms_norm(r + attention(r), w[p + "input_layernorm.weight"], eps)
            r = plain.rms_norm(r + feed_forward(r), w[p + "post_attention_layernorm.weight"], eps)
        else:
            r = r + attention(plain.rms_norm(r, w[p + "input_layernorm.weight"], eps))
            r = r + feed_forward(plain.rms_norm(r, w[p + "post_attention_layernorm.weight"], eps))
    head = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings") else w["lm_head.weight"]
    return plain.rms_norm(r, w["model.norm.weight"], eps) @ head.T


@pytest.mark.parametrize("cfg,seed", [(TINY_A, 0), (TINY_B, 1)])
def test_each_pin_rejects_the_misreading_it_is_there_for(cfg, seed):
    w = _random_weights(cfg, seed)
    toks = torch.randint(0, cfg["vocab_size"], (19,), generator=torch.Generator().manual_seed(seed)).tolist()
    # the function with its switches off is the plain implementation
    torch.testing.assert_close(_variant_logits(cfg, w, toks), plain.logits(cfg, w, toks), rtol=1e-5, atol=1e-6)

    # 1. q/k norm before the rotation. The norm's weight differs from entry to entry, so a norm *after* the rotation
    # mixes the turned pairs with unequal weights and the scores depend on where the sequence starts: the pin
    # "only distances between positions count" holds for the right order and fails for the wrong one.
    def shift_error(**switches):
        return (_variant_logits(cfg, w, toks, first_position=0, **switches)
                - _variant_logits(cfg, w, toks, first_position=37, **switches)).abs().max().item()
    assert shift_error() < 2e-5
    assert shift_error(norm_after_rotation=True) > 50 * 2e-5

    # 2. the pre-norm block with the addition carried to the next norm: with every layer's output projections at
    # zero the residual stream stays the embedding and the logits are norm(embedding) . head^T. A post-norm block
    # norms the stream itself in every layer and gives other logits.
    dead = {n: (torch.zeros_like(t) if n.endswith(("o_proj.weight", "down_proj.weight")) else t) for n, t in w.items()}
    e = w["model.embed_tokens.weight"]
    head = e if cfg.get("tie_word_embeddings") else w["lm_head.weight"]
    ref = F.rms_norm(e[toks], (cfg["hidden_size"],), w["model.norm.weight"], cfg["rms_norm_eps"]) @ head.T
    torch.testing.assert_close(_variant_logits(cfg, dead, toks), ref, rtol=1e-5, atol=1e-6)
    assert (_variant_logits(cfg, dead, toks, post_norm=True) - ref).abs().max() > 1e-2

    # 3. the scale is head_dim ** -0.5, which is the library routine's own default: attention of whole heads without
    # rotation equals F.scaled_dot_product_attention called *without* a scale; another power of the head size does not
    D = cfg["head_dim"]
    g = torch.Generator().manual_seed(seed)
    q, k, v = (torch.randn(11, 3, D, generator=g) for _ in range(3))
    lib = F.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1), is_causal=True).transpose(0, 1)
    torch.testing.assert_close(plain.causal_attention(q, k, v, D ** -0.5), lib, rtol=1e-5, atol=1e-6)
    assert (plain.causal_attention(q, k, v, D ** -1.0) - lib).abs().max() > 1e-2
    assert (_variant_logits(cfg, w, toks, scale_power=-1.0) - plain.logits(cfg, w, toks)).abs().max() > 1e-4

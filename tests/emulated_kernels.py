"""A stand-in for the HIP library, in torch on the CPU, for tests without a GPU.

It lets the engine's own logic (batch layout, block tables, slot mapping, cache
reuse, scheduling) be tested where no GPU exists. It is not a path of the
product: the engine never selects it; only tests install it with
``ops.set_backend``. Each method does what the kernel of the same name does.
"""
from __future__ import annotations

import torch


class EmulatedBackend:
    name = "emulated"
    device_type = "cpu"

    def embed(self, ids, table, out, scale=1.0):
        rows = table[ids.long()]
        out.copy_(rows if scale == 1.0 else (rows.float() * scale).to(out.dtype))

    def soft_cap(self, x, cap):
        x.copy_(cap * torch.tanh(x / cap))

    def rmsnorm(self, x, residual, residual_mode, w, y, eps):
        s = x.float()
        if residual_mode == 1:
            s = s + residual.float()
        if residual_mode != 0:
            residual.copy_(s.to(residual.dtype))
        r = torch.rsqrt(s.pow(2).mean(-1, keepdim=True) + eps)
        y.copy_(((s * r).to(x.dtype).float() * w.float()).to(x.dtype))

    def silu_mul(self, gu, out):
        I = out.shape[1]
        g, u = gu[:, :I].float(), gu[:, I:].float()
        out.copy_((g * torch.sigmoid(g) * u).to(out.dtype))

    def gather_rows(self, x, rows, out):
        out.copy_(x[rows.long()])

    def qk_rope_write(self, qkv, bias, q_norm_w, k_norm_w, eps, cos_sin, rot, positions, slot_mapping,
                      q_out, k_cache, v_cache, Hq, Hkv, D, write_kv, pair_axes=None):
        T = qkv.shape[0]
        dt = qkv.dtype
        x = qkv.float()
        if bias is not None:
            x = (x + bias.float()).to(dt).float()
        q = x[:, :Hq * D].reshape(T, Hq, D)
        k = x[:, Hq * D:(Hq + Hkv) * D].reshape(T, Hkv, D)
        v = x[:, (Hq + Hkv) * D:].reshape(T, Hkv, D)

        def norm(t, w):
            r = torch.rsqrt(t.pow(2).mean(-1, keepdim=True) + eps)
            return ((t * r).to(dt).float() * w.float()).to(dt).float()

        def turn(t):
            if rot == 0:
                return t
            if positions.dim() == 1:
                cs = cos_sin[positions.long()]                # [T, rot]
                cos, sin = cs[:, None, :rot // 2], cs[:, None, rot // 2:]
            else:
                # pair j turns by the coordinate of its axis (axis 0 where no axes are named)
                axes = pair_axes.long() if pair_axes is not None else torch.zeros(rot // 2, dtype=torch.long)
                at = positions.long()[axes].T                 # [T, rot/2]: the position that turns each pair
                j = torch.arange(rot // 2)
                cos, sin = cos_sin[at, j][:, None, :], cos_sin[at, j + rot // 2][:, None, :]
            t1, t2 = t[..., :rot // 2], t[..., rot // 2:rot]
            return torch.cat((t1 * cos - t2 * sin, t2 * cos + t1 * sin, t[..., rot:]), dim=-1)

        if q_norm_w is not None:
            q, k = norm(q, q_norm_w), norm(k, k_norm_w)
        q_out.copy_(turn(q).to(dt))
        if write_kv:
            k = turn(k).to(dt)
            ok = slot_mapping >= 0
            slots = slot_mapping[ok].long()
            k_cache.view(-1, Hkv, D)[slots] = k[ok]
            v_cache.view(-1, Hkv, D)[slots] = v[ok].to(dt)

    def paged_attention(self, q, k_cache, v_cache, out, batch, block_tables, scale, window):
        T, Hq, D = q.shape
        page_size, Hkv = k_cache.shape[1], k_cache.shape[2]
        group = Hq // Hkv
        kf = k_cache.view(-1, Hkv, D)
        vf = v_cache.view(-1, Hkv, D)
        for t in range(T):
            r = int(batch.token_req[t])
            p = int(batch.positions[t])
            lo = max(0, p - window + 1) if window > 0 else 0
            kp = torch.arange(lo, p + 1)
            slots = block_tables[r, kp // page_size].long() * page_size + kp % page_size
            for h in range(Hq):
                kh = kf[slots, h // group].float()
                vh = vf[slots, h // group].float()
                s = (kh @ q[t, h].float()) * scale
                out[t, h] = (torch.softmax(s, dim=0) @ vh).to(out.dtype)

    def linear(self, x, w, bias, out):
        y = x.float() @ w.float().T
        if bias is not None:
            y = y + bias.float()
        out.copy_(y.to(out.dtype))

    # products of few rows that take over the residual addition after them and the norm before them
    few_rows = 16
    fuse_norms = True

    def fused_linear(self, x, w, bias, out, gated=False, row_scales=None, residual=None, sum_out=None, ss_out=None, next_w=None):
        dt = x.dtype
        y = x.float() @ w.float().T
        if row_scales is not None:
            ss, eps = row_scales
            y = y * torch.rsqrt(ss.sum(-1, keepdim=True) / x.shape[1] + eps)
        if gated:
            half = w.shape[0] // 2
            g, u = y[:, :half], y[:, half:]
            y = g * torch.sigmoid(g) * u
        elif bias is not None:
            y = y + bias.float()
        if residual is None:
            out.copy_(y.to(out.dtype))
            return
        s = y + residual.float()
        residual.copy_(s.to(residual.dtype))
        sum_out.copy_((s * (next_w.float() if next_w is not None else 1.0)).to(dt))
        pad = (-s.shape[1]) % 16
        ss_out.copy_(torch.nn.functional.pad(s * s, (0, pad)).view(s.shape[0], -1, 16).sum(-1))

    def scale_rows(self, x, squares, eps, out):
        r = torch.rsqrt(squares.sum(-1, keepdim=True) / x.shape[1] + eps)
        out.copy_((x.float() * r).to(out.dtype))

    def sample(self, logits, temperatures, keys, tokens):
        from plain_qwen3 import sample_token
        import math
        mask = (1 << 64) - 1

        def mix(z):
            z = (z + 0x9E3779B97F4A7C15) & mask
            z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & mask
            z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & mask
            return z ^ (z >> 31)

        for r in range(logits.shape[0]):
            temp = float(temperatures[r])
            noise = None
            if temp > 0:
                key = int(keys[r]) & mask
                noise = torch.tensor([-math.log(((mix(key ^ i) >> 40) + 0.5) / 16777216.0)
                                      for i in range(logits.shape[1])], dtype=torch.float32)
            tokens[r] = sample_token(logits[r], temp, noise)

"""Every HIP kernel alone against a plain torch float32 reference of the same
operation, at sizes other than the tiny models' (widths and vocabularies that are
no power of two, odd head counts, head sizes in steps of 16, page sizes that do not
divide the lengths). Pure data movement must be bit-exact."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


def tol(dtype):
    # float32: rounding of a few float operations; bfloat16: one rounding to 8 bits (2^-9 relative) of
    # values of size about 1-4
    return dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=1.6e-2, atol=1.6e-2)


@pytest.fixture(scope="module")
def ops():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from nanohybrid_vlm_amd.native import ops as o
    assert o.backend().name == "hip"
    return o


def rnd(*shape, dtype=torch.float32, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).cuda()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,H,V", [(1, 80, 301), (37, 1000, 77), (300, 4096, 1000)])
def test_embed_and_gather_are_exact(ops, dtype, T, H, V):
    table = rnd(V, H, dtype=dtype)
    ids = torch.randint(0, V, (T,), dtype=torch.int32, device="cuda")
    out = ops.embed(ids, table)
    assert torch.equal(out, table[ids.long()])
    rows = torch.randint(0, T, (5,), dtype=torch.int32, device="cuda")
    assert torch.equal(ops.gather_rows(out, rows), out[rows.long()])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,H,eps", [(3, 80, 1e-5), (17, 1000, 1e-6), (5, 4096, 1e-6), (2, 12288, 1e-3), (4, 1001, 1e-5),
                                     (1, 8192, 1e-6), (300, 5120, 1e-6), (2, 16368, 1e-6)])
def test_rmsnorm(ops, dtype, T, H, eps):
    x = rnd(T, H, dtype=dtype, seed=1, scale=3.0)
    w = (1 + 0.1 * torch.randn(H)).to(dtype).cuda()
    y = ops.rmsnorm(x, w, eps)
    xf = x.float()
    ref = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * w.float()
    torch.testing.assert_close(y.float(), ref, **tol(dtype))
    # with a residual: the carried sum is the rounded sum; the norm is of the unrounded one
    res = rnd(T, H, dtype=dtype, seed=2, scale=3.0)
    res_before = res.clone()
    y2 = ops.rmsnorm(x, w, eps, residual=res)
    s = x.float() + res_before.float()
    assert torch.equal(res, s.to(dtype))
    ref2 = s * torch.rsqrt(s.pow(2).mean(-1, keepdim=True) + eps) * w.float()
    torch.testing.assert_close(y2.float(), ref2, **tol(dtype))


def test_rmsnorm_float32_residual_with_bfloat16_rows(ops):
    """The residual carried in float32: started from x exactly, then sums are not rounded."""
    x = rnd(6, 200, dtype=torch.bfloat16, seed=1)
    w = (1 + 0.1 * torch.randn(200)).bfloat16().cuda()
    y, res = ops.rmsnorm(x, w, 1e-6, start_residual=True)
    assert res.dtype == torch.float32 and torch.equal(res, x.float())
    torch.testing.assert_close(y.float(), ops.rmsnorm(x, w, 1e-6).float(), rtol=0, atol=0)
    x2 = rnd(6, 200, dtype=torch.bfloat16, seed=2)
    y2 = ops.rmsnorm(x2, w, 1e-6, residual=res)
    s = x.float() + x2.float()
    assert torch.equal(res, s)
    ref = s * torch.rsqrt(s.pow(2).mean(-1, keepdim=True) + 1e-6) * w.float()
    torch.testing.assert_close(y2.float(), ref, **tol(torch.bfloat16))
    # the residual in the rows' own type: it starts as x itself, and a sum is rounded when it is stored
    y3, res3 = ops.rmsnorm(x, w, 1e-6, start_residual=True, residual_float32=False)
    assert res3 is x and torch.equal(y3, y)
    before = x.clone()
    y4 = ops.rmsnorm(x2, w, 1e-6, residual=res3)
    assert torch.equal(res3, (before.float() + x2.float()).bfloat16())
    torch.testing.assert_close(y4.float(), ref, **tol(torch.bfloat16))


def test_rmsnorm_float32_weight_with_bfloat16_rows(ops):
    x = rnd(4, 96, dtype=torch.bfloat16)
    w = (1 + 0.1 * torch.randn(96)).cuda()
    y = ops.rmsnorm(x, w, 1e-6)
    xf = x.float()
    ref = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-6)).bfloat16().float() * w
    torch.testing.assert_close(y.float(), ref, **tol(torch.bfloat16))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,I", [(1, 112), (33, 1001), (64, 12288)])
def test_silu_mul(ops, dtype, T, I):
    gu = rnd(T, 2 * I, dtype=dtype, seed=3, scale=2.0)
    out = ops.silu_mul(gu)
    g, u = gu[:, :I].float(), gu[:, I:].float()
    torch.testing.assert_close(out.float(), torch.nn.functional.silu(g) * u, **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,N,K", [(1, 301, 80), (7, 389, 96), (65, 130, 1000), (128, 256, 512), (3, 1000, 4104)])
def test_linear(ops, dtype, M, N, K):
    x = rnd(M, K, dtype=dtype, seed=4)
    w = rnd(N, K, dtype=dtype, seed=5, scale=K ** -0.5)
    b = rnd(N, dtype=dtype, seed=6)
    ref = x.double() @ w.double().T
    t = dict(rtol=1e-5, atol=2e-5) if dtype == torch.float32 else tol(dtype)
    torch.testing.assert_close(ops.linear(x, w).double(), ref, **t)
    torch.testing.assert_close(ops.linear(x, w, b).double(), ref + b.double(), **t)
    if dtype == torch.bfloat16:
        # float32 output from bfloat16 inputs (the logits): only the accumulation rounds
        torch.testing.assert_close(ops.linear(x, w, out_dtype=torch.float32).double(), ref, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("residual_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("norm_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,H,N", [(1, 4096, 6144), (8, 4096, 1536), (16, 1024, 389), (5, 96, 80), (16, 12288, 512), (7, 5120, 4096),
                                   (3, 72, 40), (16, 1000, 24), (12, 2056, 130)])      # widths that end inside a tile of 16
def test_products_that_take_over_the_addition_and_the_norm(ops, M, H, N, norm_dtype, residual_dtype):
    """``linear(x, w, add_to=AddTo(residual, norm weight, eps))`` of few rows adds its result to the residual stream
    in its own kernel and leaves the sum times the norm's weight, rounded, and the tiles' shares of the rows' sums
    of squares (``Summed``); what is left of the norm, the scaling of the rows, is done by the product that reads
    ``Normed(summed)``, on its finished sums. Both against the same steps in float64: residual += x w1^T;
    y = rmsnorm(residual) w2^T (plain and gated)."""
    K1 = 256
    x = rnd(M, K1, dtype=torch.bfloat16, seed=31)
    w1 = rnd(H, K1, dtype=torch.bfloat16, seed=32, scale=K1 ** -0.5)
    residual = rnd(M, H, dtype=residual_dtype, seed=33)
    before = residual.clone()
    norm_w = (1 + 0.1 * torch.randn(H)).to(norm_dtype).cuda()
    w2 = rnd(N, H, dtype=torch.bfloat16, seed=34, scale=H ** -0.5)
    w3 = rnd(2 * (N // 2), H, dtype=torch.bfloat16, seed=35, scale=H ** -0.5)
    bias = rnd(N, dtype=torch.bfloat16, seed=37)
    eps = 1e-5
    summed = ops.linear(x, w1, add_to=ops.AddTo(residual, norm_w, eps))
    assert isinstance(summed, ops.Summed) and summed.residual is residual and summed.norm_weight is norm_w
    want_sum = before.double() + x.double() @ w1.double().T
    torch.testing.assert_close(residual.double(), want_sum, **(dict(rtol=1e-5, atol=1e-5) if residual_dtype == torch.float32 else tol(torch.bfloat16)))
    torch.testing.assert_close(summed.weighted.double(), want_sum * norm_w.double(), **tol(torch.bfloat16))
    assert summed.squares.shape == (M, (H + 15) // 16)
    torch.testing.assert_close(summed.squares.double().sum(-1), want_sum.pow(2).sum(-1), rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(summed.squares[:, 3].double(), want_sum[:, 48:64].pow(2).sum(-1), rtol=1e-4, atol=1e-4)
    # the scaling left to the products that read it
    normed = ops.Normed(summed)
    scale = torch.rsqrt(want_sum.pow(2).mean(-1, keepdim=True) + eps)
    want_normed = want_sum * scale * norm_w.double()
    torch.testing.assert_close(normed.tensor().double(), want_normed, **tol(torch.bfloat16))
    # (the products are compared with products of the weighted sum as it was rounded, scaled afterwards: what is left
    # is the order of the sums)
    rows = summed.weighted.double()
    y = ops.linear(normed, w2, bias)
    torch.testing.assert_close(y.double(), rows @ w2.double().T * scale + bias.double(), **tol(torch.bfloat16))
    torch.testing.assert_close(y.double(), want_normed @ w2.double().T + bias.double(), rtol=3e-2, atol=3e-2)
    g = rows @ w3.double().T * scale
    half = w3.shape[0] // 2
    torch.testing.assert_close(ops.gated_linear(normed, w3).double(),
                               torch.nn.functional.silu(g[:, :half]) * g[:, half:], **tol(torch.bfloat16))
    # and one product that does both: the scaling of its rows and the addition of its result
    res2 = rnd(M, N, dtype=residual_dtype, seed=36)
    before2 = res2.clone()
    next_w = (1 + 0.1 * torch.randn(N)).to(norm_dtype).cuda()
    both = ops.linear(normed, w2, add_to=ops.AddTo(res2, next_w, eps))
    assert isinstance(both, ops.Summed)
    torch.testing.assert_close(both.weighted.double(), (before2.double() + rows @ w2.double().T * scale) * next_w.double(),
                               **tol(torch.bfloat16))
    # switched off, the same calls give tensors and leave the residual alone
    backend = ops.backend()
    backend.fuse_norms = False
    try:
        res3 = before.clone()
        plain = ops.linear(x, w1, add_to=ops.AddTo(res3, norm_w, eps))
        assert isinstance(plain, torch.Tensor) and torch.equal(res3, before)
        torch.testing.assert_close(plain.double(), x.double() @ w1.double().T, **tol(torch.bfloat16))
        torch.testing.assert_close(ops.linear(normed, w2).double(), want_normed @ w2.double().T, rtol=3e-2, atol=3e-2)
    finally:
        backend.fuse_norms = True


@pytest.mark.parametrize("M,N,K", [(1, 4096, 4096), (8, 1000, 12288), (16, 389, 96), (17, 301, 80), (33, 6144, 1024),
                                   (48, 50, 2048), (64, 151936, 256), (64, 4096, 12288)])
def test_skinny_linear_bfloat16(ops, M, N, K):
    """Few rows in bfloat16 (a decoding step): own MFMA kernel, K split over waves."""
    x = rnd(M, K, dtype=torch.bfloat16, seed=14)
    w = rnd(N, K, dtype=torch.bfloat16, seed=15, scale=K ** -0.5)
    ref = x.double() @ w.double().T
    torch.testing.assert_close(ops.linear(x, w, out_dtype=torch.float32).double(), ref, rtol=1e-4, atol=2e-4)
    torch.testing.assert_close(ops.linear(x, w).double(), ref, **tol(torch.bfloat16))
    # inside a HIP graph no library is called: the own kernel also takes 17 to 64 rows with bfloat16 output
    backend = ops.backend()
    backend.own_kernels_only = True
    try:
        torch.testing.assert_close(ops.linear(x, w).double(), ref, **tol(torch.bfloat16))
    finally:
        backend.own_kernels_only = False
    # a row's result does not depend on how many other rows there are, beyond the rounding of the float sums
    # (the number of waves that split K changes with the number of rows)
    if M > 1:
        torch.testing.assert_close(ops.linear(x[:1].contiguous(), w, out_dtype=torch.float32),
                                   ops.linear(x, w, out_dtype=torch.float32)[:1], rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("M,N,K", [
    # every way the kernel for up to 16 rows cuts the work: one or two tiles of 16 outputs per block, 4 or 8 waves
    (1, 6144, 264), (2, 5000, 4096), (5, 7168, 72), (8, 6100, 1032), (12, 5120, 520), (16, 151936, 64), (9, 10240, 40),
    (16, 16, 8), (3, 17, 25608),
    # x too large for LDS at once, up to 256 tiles: it comes in pieces
    (16, 4000, 12296), (7, 272, 12288), (11, 4096, 25600),
    # x too large for LDS at once and more than 256 tiles: two pieces, every tile walked over twice
    (16, 7168, 5120), (10, 5136, 8200), (5, 4112, 17408),
])
def test_few_rows_linear_bfloat16_in_all_its_variants(ops, M, N, K):
    x = rnd(M, K, dtype=torch.bfloat16, seed=34)
    w = rnd(N, K, dtype=torch.bfloat16, seed=35, scale=K ** -0.5)
    b = rnd(N, dtype=torch.bfloat16, seed=36)
    ref = x.double() @ w.double().T
    torch.testing.assert_close(ops.linear(x, w, out_dtype=torch.float32).double(), ref, rtol=1e-4, atol=2e-4)
    torch.testing.assert_close(ops.linear(x, w, b).double(), ref + b.double(), **tol(torch.bfloat16))
    # the same call twice gives the same bits: the sums are added in a fixed order
    assert torch.equal(ops.linear(x, w, out_dtype=torch.float32), ops.linear(x, w, out_dtype=torch.float32))


@pytest.mark.parametrize("M,I,K", [(1, 112, 80), (5, 1001, 96), (16, 12288, 4096), (17, 160, 96), (64, 300, 1024),
                                   (4, 17408, 136), (16, 25600, 72), (13, 25000, 264), (16, 9000, 5120), (15, 520, 5384)])
def test_gated_linear(ops, M, I, K):
    """silu(x Wg^T) * (x Wu^T): the fused kernel for few rows, the two-kernel way for many; float32 as well."""
    for dtype in DTYPES:
        x = rnd(M, K, dtype=dtype, seed=24)
        w = rnd(2 * I, K, dtype=dtype, seed=25, scale=K ** -0.5)
        g, u = x.double() @ w[:I].double().T, x.double() @ w[I:].double().T
        ref = g * torch.sigmoid(g) * u
        t = dict(rtol=1e-5, atol=2e-5) if dtype == torch.float32 else tol(dtype)
        torch.testing.assert_close(ops.gated_linear(x, w).double(), ref, **t)
        backend = ops.backend()
        backend.own_kernels_only = True                      # as inside a HIP graph: fused up to 64 rows
        try:
            torch.testing.assert_close(ops.gated_linear(x, w).double(), ref, **t)
        finally:
            backend.own_kernels_only = False


def test_linear_rows_do_not_depend_on_the_batch_in_float32(ops):
    x = rnd(70, 200, seed=7)
    w = rnd(150, 200, seed=8)
    full = ops.linear(x, w)
    for rows in ([0], [69], [3, 4, 5], list(range(64, 70))):
        part = ops.linear(x[rows].contiguous(), w)
        assert torch.equal(part, full[rows])


def _rope_reference(x, positions, base, rot):
    inv = 1.0 / (base ** (torch.arange(0, rot, 2, dtype=torch.float32) / rot))
    ang = positions.float()[:, None] * inv[None, :]
    cos, sin = ang.cos()[:, None, :], ang.sin()[:, None, :]
    x1, x2 = x[..., :rot // 2], x[..., rot // 2:rot]
    return torch.cat((x1 * cos - x2 * sin, x2 * cos + x1 * sin, x[..., rot:]), dim=-1)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("Hq,Hkv,D,rot,norm,bias", [
    (4, 2, 16, 16, True, False), (6, 1, 32, 32, True, False), (5, 5, 48, 48, False, True),
    (3, 3, 80, 40, True, False), (32, 8, 128, 128, True, False), (2, 1, 256, 0, False, False),
])
def test_qk_rope_write(ops, dtype, Hq, Hkv, D, rot, norm, bias):
    from nanohybrid_vlm_amd.parts.positions import RotaryEmbedding
    T, page, pages, eps, base = 23, 8, 9, 1e-5, 10000.0
    width = (Hq + 2 * Hkv) * D
    qkv = rnd(T, width, dtype=dtype, seed=9, scale=2.0)
    b = rnd(width, dtype=dtype, seed=10) if bias else None
    qw = (1 + 0.1 * torch.randn(D)).to(dtype).cuda() if norm else None
    kw = (1 + 0.1 * torch.randn(D)).to(dtype).cuda() if norm else None
    table = RotaryEmbedding(rot, 300, base).table.cuda() if rot else None
    positions = torch.randint(0, 300, (T,), dtype=torch.int32, device="cuda")
    slots = torch.randperm(page * pages)[:T].to(torch.int32).cuda()
    slots[5] = -1                                     # a token that is not stored
    k_cache = torch.zeros(pages, page, Hkv, D, dtype=dtype, device="cuda")
    v_cache = torch.zeros_like(k_cache)
    q = ops.qk_rope_write(qkv, b, qw, kw, eps, table, positions, slots, k_cache, v_cache, Hq, Hkv, D)

    x = qkv.float()
    if bias:
        x = (x + b.float()).to(dtype).float()
    qr = x[:, :Hq * D].reshape(T, Hq, D)
    kr = x[:, Hq * D:(Hq + Hkv) * D].reshape(T, Hkv, D)
    vr = x[:, (Hq + Hkv) * D:].reshape(T, Hkv, D)
    if norm:
        qr = qr * torch.rsqrt(qr.pow(2).mean(-1, keepdim=True) + eps) * qw.float()
        kr = kr * torch.rsqrt(kr.pow(2).mean(-1, keepdim=True) + eps) * kw.float()
    if rot:
        qr = _rope_reference(qr.cpu(), positions.cpu(), base, rot).cuda()
        kr = _rope_reference(kr.cpu(), positions.cpu(), base, rot).cuda()
    t = tol(dtype) if dtype == torch.bfloat16 else dict(rtol=1e-5, atol=2e-5)
    torch.testing.assert_close(q.float(), qr, **t)
    stored = slots >= 0
    kf, vf = k_cache.view(-1, Hkv, D), v_cache.view(-1, Hkv, D)
    torch.testing.assert_close(kf[slots[stored].long()].float(), kr[stored], **t)
    assert torch.equal(vf[slots[stored].long()], vr[stored].to(dtype))      # values are only moved
    untouched = torch.ones(page * pages, dtype=torch.bool, device="cuda")
    untouched[slots[stored].long()] = False
    assert not kf[untouched].any() and not vf[untouched].any()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("Hq,Hkv,D,rot,axes", [(4, 2, 16, 16, 2), (3, 1, 48, 24, 3), (8, 2, 128, 128, 2), (2, 2, 32, 8, 1)])
def test_qk_rope_write_over_several_position_axes(ops, dtype, Hq, Hkv, D, rot, axes):
    """positions [axes, T]: pair j of a head turns by the angle that the table holds at the coordinate of axis
    pair_axes[j] (without pair_axes: of the first axis)."""
    from nanohybrid_vlm_amd.parts.positions import RotaryEmbedding
    T, base = 19, 10000.0
    width = (Hq + 2 * Hkv) * D
    qkv = rnd(T, width, dtype=dtype, seed=19, scale=2.0)
    table = RotaryEmbedding(rot, 200, base).table.cuda()
    positions = torch.randint(0, 200, (axes, T), dtype=torch.int32, device="cuda")
    pair_axes = (torch.arange(rot // 2) * 5 % axes).to(torch.int32).cuda() if axes > 1 else None
    slots = torch.arange(T, dtype=torch.int32, device="cuda")
    k_cache = torch.zeros(4, 8, Hkv, D, dtype=dtype, device="cuda")
    v_cache = torch.zeros_like(k_cache)
    q = ops.qk_rope_write(qkv, None, None, None, 0.0, table, positions, slots, k_cache, v_cache, Hq, Hkv, D, pair_axes=pair_axes)
    # the angle of pair j at position p is p * base^(-2j/rot): here p differs from pair to pair
    j = torch.arange(rot // 2)
    at = positions.cpu().long()[pair_axes.cpu().long() if pair_axes is not None else torch.zeros(rot // 2, dtype=torch.long)].T   # [T, rot/2]
    ang = at.double() * (base ** (-2.0 * j.double() / rot))
    cos, sin = ang.cos()[:, None, :], ang.sin()[:, None, :]

    def turned(x):
        x = x.double().cpu()
        x1, x2 = x[..., :rot // 2], x[..., rot // 2:rot]
        return torch.cat((x1 * cos - x2 * sin, x2 * cos + x1 * sin, x[..., rot:]), -1)

    x = qkv.float()
    t = dict(rtol=1.6e-2, atol=1.6e-2) if dtype == torch.bfloat16 else dict(rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(q.double().cpu(), turned(x[:, :Hq * D].reshape(T, Hq, D)), **t)
    torch.testing.assert_close(k_cache.view(-1, Hkv, D)[:T].double().cpu(), turned(x[:, Hq * D:(Hq + Hkv) * D].reshape(T, Hkv, D)), **t)


@pytest.mark.parametrize("dtype", DTYPES)
def test_embed_scale_and_soft_cap(ops, dtype):
    table = rnd(301, 200, dtype=dtype, seed=21)
    ids = torch.randint(0, 301, (13,), dtype=torch.int32, device="cuda")
    assert torch.equal(ops.embed(ids, table, 1.0), table[ids.long()])
    assert torch.equal(ops.embed(ids, table, 1.75), (table[ids.long()].float() * 1.75).to(dtype))
    logits = rnd(7, 1001, seed=22, scale=6.0)
    want = 4.0 * torch.tanh(logits / 4.0)
    assert ops.soft_cap_(logits, 4.0) is logits
    torch.testing.assert_close(logits, want, rtol=1e-5, atol=1e-5)
    assert float(logits.abs().max()) <= 4.0


def _paged_setup(dtype, lens, q_lens, Hq, Hkv, D, page, seed=0, scale=1.0):
    """Requests with ``lens`` keys each whose last ``q_lens`` tokens are this step's queries; pages handed out
    in a shuffled order. Returns the pieces for ops.paged_attention and the dense keys and values."""
    from nanohybrid_vlm_amd.native.ops import AttentionBatch
    g = torch.Generator().manual_seed(seed)
    B = len(lens)
    n_pages = sum(-(-n // page) for n in lens) + 3
    order = torch.randperm(n_pages, generator=g).tolist()
    k_cache = torch.full((n_pages, page, Hkv, D), float("nan"), dtype=dtype)
    v_cache = torch.full((n_pages, page, Hkv, D), float("nan"), dtype=dtype)
    width = max(-(-n // page) for n in lens)
    bt = torch.full((B, width), -1, dtype=torch.int32)
    ks, vs, qs, token_req, positions = [], [], [], [], []
    for r, (n, nq) in enumerate(zip(lens, q_lens)):
        k = (torch.randn(n, Hkv, D, generator=g) * scale).to(dtype)
        v = torch.randn(n, Hkv, D, generator=g).to(dtype)
        ks.append(k)
        vs.append(v)
        for lp in range(-(-n // page)):
            pid = order.pop()
            bt[r, lp] = pid
            m = min(page, n - lp * page)
            k_cache[pid, :m] = k[lp * page:lp * page + m]
            v_cache[pid, :m] = v[lp * page:lp * page + m]
        qs.append((torch.randn(nq, Hq, D, generator=g) * scale).to(dtype))
        token_req += [r] * nq
        positions += list(range(n - nq, n))
    cu = torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32)
    batch = AttentionBatch(num_tokens=sum(q_lens), num_requests=B,
                           token_req=torch.tensor(token_req, dtype=torch.int32).cuda(),
                           positions=torch.tensor(positions, dtype=torch.int32).cuda(),
                           cu_seqlens_q=cu.cuda(), context_lens=torch.tensor(lens, dtype=torch.int32).cuda(),
                           max_q_len=max(q_lens), max_context_len=max(lens))
    return torch.cat(qs).cuda(), k_cache.cuda(), v_cache.cuda(), batch, bt.cuda(), ks, vs, qs


def _attention_reference(qs, ks, vs, lens, q_lens, scale, window):
    outs = []
    for q, k, v, n, nq in zip(qs, ks, vs, lens, q_lens):
        Hq, Hkv = q.shape[1], k.shape[1]
        kk = k.double().repeat_interleave(Hq // Hkv, dim=1)
        vv = v.double().repeat_interleave(Hq // Hkv, dim=1)
        s = torch.einsum("qhd,khd->hqk", q.double(), kk) * scale
        qpos = torch.arange(n - nq, n)[:, None]
        kpos = torch.arange(n)[None, :]
        ok = kpos <= qpos
        if window:
            ok &= kpos > qpos - window
        s = s.masked_fill(~ok[None], float("-inf"))
        outs.append(torch.einsum("hqk,khd->qhd", torch.softmax(s, dim=-1), vv))
    return torch.cat(outs)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("Hq,Hkv,D,page,window", [
    (4, 2, 16, 4, None), (6, 1, 32, 8, None), (5, 5, 48, 7, None), (3, 1, 80, 16, 9),
    (8, 2, 128, 64, None), (32, 8, 128, 256, None), (2, 2, 64, 5, 64), (7, 7, 112, 3, None),
])
def test_paged_attention(ops, dtype, Hq, Hkv, D, page, window):
    # whole prompts, portions with earlier keys, single decoded tokens, a length of one, page edges
    lens = [1, 64, 65, 300, 17, 128, 5, 257]
    q_lens = [1, 64, 1, 43, 2, 1, 5, 1]
    scale = D ** -0.5
    q, kc, vc, batch, bt, ks, vs, qs = _paged_setup(dtype, lens, q_lens, Hq, Hkv, D, page, seed=11, scale=1.5)
    out = ops.paged_attention(q, kc, vc, batch, bt, scale, window)
    ref = _attention_reference(qs, ks, vs, lens, q_lens, scale, window)
    t = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else tol(dtype)
    torch.testing.assert_close(out.double().cpu(), ref, **t)


@pytest.mark.parametrize("Hq,Hkv,D,page,window", [
    (4, 2, 16, 4, None), (6, 1, 32, 8, None), (5, 5, 48, 7, None), (3, 1, 80, 16, 9), (8, 2, 128, 64, None),
    (32, 8, 128, 256, None), (16, 1, 64, 5, 70), (7, 7, 112, 3, None), (2, 1, 256, 32, None), (12, 2, 96, 16, 300),
])
def test_decode_attention_bfloat16(ops, Hq, Hkv, D, page, window):
    """Single tokens of several requests in bfloat16: the split-key kernel (lengths around the edges of
    tiles of 16, of splits and of pages)."""
    lens = [1, 15, 16, 17, 31, 32, 33, 64, 65, 300, 257, 1000, 1024, 1025]
    q_lens = [1] * len(lens)
    scale = D ** -0.5
    q, kc, vc, batch, bt, ks, vs, qs = _paged_setup(torch.bfloat16, lens, q_lens, Hq, Hkv, D, page, seed=21, scale=1.5)
    out = ops.paged_attention(q, kc, vc, batch, bt, scale, window)
    ref = _attention_reference(qs, ks, vs, lens, q_lens, scale, window)
    torch.testing.assert_close(out.double().cpu(), ref, **tol(torch.bfloat16))
    # the same tokens one at a time (other split lengths are chosen then): same result up to rounding
    one = ops.paged_attention(q[9:10].contiguous(), kc, vc,
                              type(batch)(1, 1, torch.zeros(1, dtype=torch.int32).cuda(), batch.positions[9:10].contiguous(),
                                          torch.tensor([0, 1], dtype=torch.int32).cuda(), batch.context_lens[9:10].contiguous(),
                                          1, lens[9]), bt[9:10].contiguous(), scale, window)
    torch.testing.assert_close(one.float(), out[9:10].float(), rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("Hq,Hkv,D,page,window", [(8, 2, 128, 256, None), (6, 1, 48, 16, None), (4, 4, 64, 64, 3000)])
def test_decode_attention_of_few_tokens_over_many_splits(ops, Hq, Hkv, D, page, window):
    """One or two requests of thousands of keys: more than 32 splits of 64 keys, which four waves merge."""
    for lens in ([5000], [4097, 2100]):
        q_lens = [1] * len(lens)
        scale = D ** -0.5
        q, kc, vc, batch, bt, ks, vs, qs = _paged_setup(torch.bfloat16, lens, q_lens, Hq, Hkv, D, page, seed=27, scale=1.5)
        out = ops.paged_attention(q, kc, vc, batch, bt, scale, window)
        ref = _attention_reference(qs, ks, vs, lens, q_lens, scale, window)
        torch.testing.assert_close(out.double().cpu(), ref, **tol(torch.bfloat16))


@pytest.mark.parametrize("D,split_len,n_splits,window", [
    (128, 64, 5, None),      # one wave, four splits a lane
    (128, 64, 20, None),     # four waves, four splits a lane; the last waves' splits lie past every position but one
    (128, 64, 40, 900),      # four waves, eight a lane, a window that leaves the first splits out
    (128, 64, 100, None),    # four waves, sixteen a lane
    (128, 64, 140, None),    # past the at-once kernels: the kernel that loops, four waves
    (64, 128, 9, None), (256, 64, 3, None), (256, 64, 30, 500), (48, 64, 33, None), (16, 64, 70, None),
])
def test_merge_of_splits_in_all_its_forms(ops, D, split_len, n_splits, window):
    """The decode kernel called with the split length and the number of splits named: every form of the merge (one
    wave or four, 4 to 16 splits a lane, and the looping kernel), with more splits than most positions reach and the
    buffers of the splits' results full of NaN beforehand, so that a split read without having been written shows."""
    import ctypes
    from nanohybrid_vlm_amd.native.ops import _ptr, _stream
    Hq, Hkv, page = 8, 2, 64
    longest = n_splits * split_len
    lens = [longest, 1, split_len, split_len + 1, longest // 2 + 3, longest - 1, 77]
    lens = [n for n in lens if n <= longest]
    q_lens = [1] * len(lens)
    scale = D ** -0.5
    q, kc, vc, batch, bt, ks, vs, qs = _paged_setup(torch.bfloat16, lens, q_lens, Hq, Hkv, D, page, seed=61, scale=1.5)
    backend = ops.backend()
    T = len(lens)
    out = torch.full((T, Hq, D), float("nan"), dtype=torch.bfloat16, device="cuda")
    part_o = torch.full((T, Hq, n_splits, D), float("nan"), dtype=torch.float32, device="cuda")
    part_ml = torch.full((T, Hq, n_splits, 2), float("nan"), dtype=torch.float32, device="cuda")
    backend._call("nhv_decode_attention_bf16", _ptr(q), _ptr(kc), _ptr(vc), _ptr(out), _ptr(part_o), _ptr(part_ml),
                  _ptr(batch.token_req), _ptr(batch.positions), _ptr(bt), bt.shape[1], T, Hq, Hkv, page,
                  ctypes.c_float(scale), window or 0, split_len, n_splits, _stream(), lib=backend.attention_lib(D))
    ref = _attention_reference(qs, ks, vs, lens, q_lens, scale, window)
    torch.testing.assert_close(out.double().cpu(), ref, **tol(torch.bfloat16))


def test_merge_of_splits_of_many_tokens(ops):
    """More than 1,024 (token, head) pairs with more splits than the at-once kernels take: the looping kernel with
    one wave."""
    import ctypes
    from nanohybrid_vlm_amd.native.ops import _ptr, _stream
    Hq, Hkv, D, page, split_len, n_splits = 16, 2, 128, 64, 64, 140
    lens = [8960] + [40 + 3 * i for i in range(69)]
    q_lens = [1] * len(lens)
    scale = D ** -0.5
    q, kc, vc, batch, bt, ks, vs, qs = _paged_setup(torch.bfloat16, lens, q_lens, Hq, Hkv, D, page, seed=62, scale=1.5)
    backend = ops.backend()
    T = len(lens)
    assert T * Hq > 1024
    out = torch.full((T, Hq, D), float("nan"), dtype=torch.bfloat16, device="cuda")
    part_o = torch.full((T, Hq, n_splits, D), float("nan"), dtype=torch.float32, device="cuda")
    part_ml = torch.full((T, Hq, n_splits, 2), float("nan"), dtype=torch.float32, device="cuda")
    backend._call("nhv_decode_attention_bf16", _ptr(q), _ptr(kc), _ptr(vc), _ptr(out), _ptr(part_o), _ptr(part_ml),
                  _ptr(batch.token_req), _ptr(batch.positions), _ptr(bt), bt.shape[1], T, Hq, Hkv, page,
                  ctypes.c_float(scale), 0, split_len, n_splits, _stream(), lib=backend.attention_lib(D))
    ref = _attention_reference(qs, ks, vs, lens, q_lens, scale, None)
    torch.testing.assert_close(out.double().cpu(), ref, **tol(torch.bfloat16))


@pytest.mark.parametrize("Hq,Hkv,D,page,window", [
    (4, 1, 128, 256, None), (8, 2, 64, 16, None), (6, 1, 32, 8, 100), (3, 3, 48, 5, None), (16, 1, 16, 64, None),
    (5, 1, 256, 32, None), (32, 8, 128, 64, 700),
])
def test_prefill_attention_bfloat16(ops, Hq, Hkv, D, page, window):
    """Long portions with and without earlier keys in bfloat16: the matrix-core kernel (tiles of 64 keys and of
    16 tokens; portions that end inside a tile; a single token beside them)."""
    lens = [700, 300, 64, 1500, 17, 129]
    q_lens = [300, 300, 1, 1025, 16, 65]
    scale = D ** -0.5
    q, kc, vc, batch, bt, ks, vs, qs = _paged_setup(torch.bfloat16, lens, q_lens, Hq, Hkv, D, page, seed=31, scale=1.5)
    out = ops.paged_attention(q, kc, vc, batch, bt, scale, window)
    ref = _attention_reference(qs, ks, vs, lens, q_lens, scale, window)
    torch.testing.assert_close(out.double().cpu(), ref, **tol(torch.bfloat16))


@pytest.mark.parametrize("far", [3, 650, 1290])
def test_prefill_attention_scores_that_outgrow_their_reference(ops, far):
    """The prompt kernel takes a row's exponentials against a reference point that stays while they stay far below
    float's range. Here one key's scores stand 110 powers of two above all others, for every query of one head: an
    early key (everything after it is tiny against the reference), a key in the middle of the portion and one near
    its end (the sums so far have to be scaled down by 2^-110 when it comes). Against the float64 computation."""
    Hq, Hkv, D, page = 4, 2, 128, 64
    scale = D ** -0.5
    lens, q_lens = [1300, 200], [700, 200]
    q, kc, vc, batch, bt, ks, vs, qs = _paged_setup(torch.bfloat16, lens, q_lens, Hq, Hkv, D, page, seed=71, scale=1.0)
    g = torch.Generator().manual_seed(6)
    direction = torch.randn(D, generator=g)
    direction = (direction / direction.norm()).to(torch.bfloat16)
    ks[0][far, 0] = 30.0 * direction                              # heads 0 and 1 read key/value head 0
    kc[int(bt[0, far // page]), far % page, 0] = ks[0][far, 0].cuda()
    qs[0][:, 1] = qs[0][:, 1] + 29.0 * direction                  # 30 x 29 / sqrt(128) = 77 = 111 powers of two
    q[:q_lens[0], 1] = qs[0][:, 1].cuda()
    out = ops.paged_attention(q, kc, vc, batch, bt, scale, None)
    ref = _attention_reference(qs, ks, vs, lens, q_lens, scale, None)
    torch.testing.assert_close(out.double().cpu(), ref, **tol(torch.bfloat16))
    # (the input does what it is meant to: a query of head 1 that sees the key puts all of its weight on it)
    first_q = lens[0] - q_lens[0]
    row = max(far - first_q, 0) + 5
    torch.testing.assert_close(ref[row, 1], vs[0][far, 0].double(), rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("window", [None, 5000])
def test_attention_over_32768_keys(ops, window):
    """Both bfloat16 attention kernels at 32,768 keys on pages of 256 (128 pages a request, hundreds of splits to
    merge, block tables past what a block keeps in LDS at smaller pages), against the float64 computation: a single
    token at the end of 32,768 keys beside one after 9,001; and portions of 130 and 64 tokens that end at 32,768
    and 20,000 keys. In every request one early key is made to stand out for one head's queries, so that a key lost
    far from the end shows."""
    Hq, Hkv, D, page = 8, 2, 128, 256
    scale = D ** -0.5
    for lens, q_lens in ([[32768, 9001], [1, 1]], [[32768, 20000], [130, 64]]):
        q, kc, vc, batch, bt, ks, vs, qs = _paged_setup(torch.bfloat16, lens, q_lens, Hq, Hkv, D, page, seed=41, scale=1.0)
        # key 777 (and key n - 4100, inside a window of 5,000) of every request points where head 3's queries point
        g = torch.Generator().manual_seed(5)
        direction = torch.randn(D, generator=g)
        direction = (direction / direction.norm()).to(torch.bfloat16)
        row = 0
        for r, (n, nq) in enumerate(zip(lens, q_lens)):
            for far in (777, n - 4100):
                ks[r][far, 0] = ks[r][far, 0] + 14.0 * direction          # head 3 reads key/value head 0
                pid = int(bt[r, far // page])
                kc[pid, far % page, 0] = ks[r][far, 0].cuda()
            qs[r][:, 3] = qs[r][:, 3] + 14.0 * direction
            q[row:row + nq, 3] = qs[r][:, 3].cuda()
            row += nq
        out = ops.paged_attention(q, kc, vc, batch, bt, scale, window)
        ref = _attention_reference(qs, ks, vs, lens, q_lens, scale, window)
        torch.testing.assert_close(out.double().cpu(), ref, **tol(torch.bfloat16))
        # (the input does what it is meant to: nearly all of the softmax's weight of head 3's last query lies on the
        # keys that stand out, so an output that agrees with the reference has found them)
        for r, n in enumerate(lens):
            scores = (ks[r][:, 0].double() @ qs[r][-1, 3].double()) * scale
            if window:
                scores[:n - window] = float("-inf")
            weight = torch.softmax(scores, 0)
            far = [n - 4100] if window else [777, n - 4100]
            assert weight[far].sum() > 0.95


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("page", [8, 64, 256])
def test_attention_finds_one_far_key(ops, dtype, page):
    """One key is made to stand out (score far above the rest): the output must be that key's value,
    wherever the key lies: first of the sequence, last of a page, first of a page, the query's own position."""
    Hq, Hkv, D, n = 8, 2, 64, 700
    for far in [0, page - 1, page, 2 * page - 1, n // 2, n - 2, n - 1]:
        g = torch.Generator().manual_seed(far)
        k = torch.randn(n, Hkv, D, generator=g) * 0.1
        v = torch.randn(n, Hkv, D, generator=g)
        q = torch.randn(1, Hq, D, generator=g) * 0.1
        direction = torch.randn(D, generator=g)
        direction = direction / direction.norm()
        k[far] += 10.0 * direction
        q[0] += 10.0 * direction                    # score of `far` is about 100 * D^-0.5 = 12.5 above the others
        from nanohybrid_vlm_amd.native.ops import AttentionBatch
        n_pages = -(-n // page)
        perm = torch.randperm(n_pages, generator=g)
        kc = torch.full((n_pages, page, Hkv, D), float("nan"))
        vc = torch.full((n_pages, page, Hkv, D), float("nan"))
        for lp in range(n_pages):
            m = min(page, n - lp * page)
            kc[perm[lp], :m] = k[lp * page:lp * page + m]
            vc[perm[lp], :m] = v[lp * page:lp * page + m]
        batch = AttentionBatch(1, 1, torch.zeros(1, dtype=torch.int32).cuda(),
                               torch.tensor([n - 1], dtype=torch.int32).cuda(),
                               torch.tensor([0, 1], dtype=torch.int32).cuda(),
                               torch.tensor([n], dtype=torch.int32).cuda(), 1, n)
        out = ops.paged_attention(q.to(dtype).cuda(), kc.to(dtype).cuda(), vc.to(dtype).cuda(), batch,
                                  perm.to(torch.int32)[None].cuda(), D ** -0.5)
        ref = _attention_reference([q.to(dtype)], [k.to(dtype)], [v.to(dtype)], [n], [1], D ** -0.5, None)
        torch.testing.assert_close(out.double().cpu(), ref, **tol(dtype))
        if far < n - 1:
            # the same query once more as the second-to-last token of a portion of two (the portion kernel)
            q2 = torch.cat((q, q)).to(dtype).cuda()
            batch2 = AttentionBatch(2, 1, torch.zeros(2, dtype=torch.int32).cuda(),
                                    torch.tensor([n - 2, n - 1], dtype=torch.int32).cuda(),
                                    torch.tensor([0, 2], dtype=torch.int32).cuda(),
                                    torch.tensor([n], dtype=torch.int32).cuda(), 2, n)
            out2 = ops.paged_attention(q2, kc.to(dtype).cuda(), vc.to(dtype).cuda(), batch2,
                                       perm.to(torch.int32)[None].cuda(), D ** -0.5)
            torch.testing.assert_close(out2[1:].double().cpu(), ref, **tol(dtype))
        # and it is mostly that one value
        kvh = torch.arange(Hq) // (Hq // Hkv)
        assert (out.float().cpu()[0] - v[far, kvh]).abs().max() < 0.5, f"far key {far} not found"


@pytest.mark.parametrize("V", [301, 389, 5000, 151936])
def test_sampling(ops, V):
    import plain_qwen3 as plain
    g = torch.Generator().manual_seed(V)
    n = 6
    logits = (torch.randn(n, V, generator=g) * 3).cuda()
    logits[0, 17] = logits[0, 200] = 50.0                # a tie: the first index wins
    temps = torch.tensor([0.0, 0.0, 0.8, 1.0, 0.3, 2.5]).cuda()
    keys = torch.tensor([0, 0, 1234567, -99, 2**62 + 5, 42], dtype=torch.int64).cuda()
    tokens = ops.sample(logits, temps, keys).cpu()
    assert tokens[0] == 17
    assert tokens[1] == logits[1].argmax().item()
    if V <= 5000:
        mask = (1 << 64) - 1
        for r in range(2, n):
            key = int(keys[r]) & mask
            # the noise of plain_qwen3.sample_noise for an already mixed key
            noise = torch.tensor([plain.noise_of_bits(_mix(key ^ i) >> 40) for i in range(V)])
            assert tokens[r] == plain.sample_token(logits[r].cpu(), float(temps[r]), noise)


def _mix(z):
    mask = (1 << 64) - 1
    z = (z + 0x9E3779B97F4A7C15) & mask
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & mask
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & mask
    return z ^ (z >> 31)


def test_noise_of_every_bit_pattern(ops):
    """All 2^24 patterns through the kernel's own noise function: the values are those of the plain formula, none is
    0 or infinite, and the share of patterns below x is the Exp(1) distribution's 1 - exp(-x) to within one and a
    half patterns, from the smallest values (3e-8) up. A noise of 1e-10 once in 2^24 draws would fail both."""
    import ctypes
    import numpy as np
    n = 1 << 24
    bits = torch.arange(n, dtype=torch.int32, device="cuda")
    out = torch.empty(n, dtype=torch.float32, device="cuda")
    lib = ops.backend().lib
    assert lib.nhv_noise_of_bits(ctypes.c_void_p(bits.data_ptr()), ctypes.c_void_p(out.data_ptr()), n,
                                 ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)) == 0
    got = out.cpu().numpy().astype(np.float64)
    want = -np.log((np.arange(n, dtype=np.float64) + 0.5) / n)
    assert np.isfinite(got).all() and got.min() > 2.9e-8
    assert np.abs(got / want - 1).max() < 1e-6
    ordered = np.sort(got)
    share = np.arange(1, n + 1) / n                       # share of patterns at or below each value
    # (half a pattern by construction, and up to as much again from rounding the larger values to float)
    assert np.abs(share - (1 - np.exp(-ordered))).max() <= 1.5 / n


def test_sampling_follows_the_distribution(ops):
    """Empirical frequencies of 4000 draws against softmax(logits / T) (chi-square, fixed keys)."""
    V, draws, temp = 12, 4000, 0.7
    logits = torch.tensor([[2.0, 1.0, 0.5, 0.0, -0.5, -1.0, 1.5, 0.2, -2.0, 0.7, 0.1, -0.3]])
    p = torch.softmax(logits[0] / temp, dim=0)
    rows = logits.repeat(draws, 1).cuda()
    keys = torch.arange(draws, dtype=torch.int64).cuda() * 7919 + 13
    tokens = ops.sample(rows, torch.full((draws,), temp).cuda(), keys).cpu()
    counts = torch.bincount(tokens.long(), minlength=V).float()
    chi2 = ((counts - draws * p) ** 2 / (draws * p)).sum().item()
    assert chi2 < 31.3, f"chi-square {chi2:.1f} with 11 degrees of freedom (0.999 quantile is 31.3)"


def test_refusals(ops):
    from nanohybrid_vlm_amd.native.ops import KernelError
    x = rnd(2, 64)
    with pytest.raises(KernelError, match="columns"):
        ops.linear(x, rnd(8, 32))
    with pytest.raises(KernelError, match="element type"):
        ops.linear(x.half(), rnd(8, 64).half())
    with pytest.raises(KernelError, match="limit"):
        ops.rmsnorm(rnd(1, 20000), rnd(20000), 1e-6)
    with pytest.raises(KernelError, match="contiguous"):
        ops.rmsnorm(rnd(4, 128)[:, ::2], rnd(64), 1e-6)
    with pytest.raises(KernelError, match="device"):
        ops.rmsnorm(torch.zeros(2, 8), torch.ones(8), 1e-6)


def test_products_of_few_rows_are_done_the_fastest_way_measured(ops):
    """While ``measure_linears`` is set a shape not seen before is timed by the own kernel and by every algorithm
    of the library, and the answer kept; whichever way a product goes, it is the same product."""
    from nanohybrid_vlm_amd.native.ops import OWN
    backend = ops.backend()
    N, K = 512, 1024
    for M in (8, 40):                                       # the own kernel is among the ways / the library's ways only
        x = rnd(M, K, dtype=torch.bfloat16, seed=51)
        w = rnd(N, K, dtype=torch.bfloat16, seed=52, scale=K ** -0.5)
        w2 = rnd(2 * N, K, dtype=torch.bfloat16, seed=53, scale=K ** -0.5)
        ref = x.double() @ w.double().T
        g, u = x.double() @ w2[:N].double().T, x.double() @ w2[N:].double().T
        keys = [(M, N, K, False, False), (M, N, K, True, False)] + ([(M, 2 * N, K, False, True)] if M <= 16 else [])
        every = keys + [(M, 2 * N, K, False, False)]
        saved = {k: backend.chosen.pop(k, None) for k in every}
        try:
            assert ops.linear(x, w) is not None and keys[0] not in backend.chosen      # not measured unasked
            backend.measure_linears = True
            try:
                ops.linear(x, w)
                ops.linear(x, w, out_dtype=torch.float32)
                ops.gated_linear(x, w2)
            finally:
                backend.measure_linears = False
                backend.end_measurements()
            assert all(isinstance(backend.chosen[k], int) for k in keys)
            assert M <= 16 or all(backend.chosen[k] != OWN for k in keys)
            _, count = backend._library_plan(M, N, K, False)
            assert count > 0
            for how in [OWN] + list(range(min(count, 3))):
                for k in every:
                    backend.chosen[k] = how
                torch.testing.assert_close(ops.linear(x, w).double(), ref, **tol(torch.bfloat16))
                torch.testing.assert_close(ops.linear(x, w, out_dtype=torch.float32).double(), ref, rtol=1e-4, atol=1e-4)
                torch.testing.assert_close(ops.gated_linear(x, w2).double(), g * torch.sigmoid(g) * u, **tol(torch.bfloat16))
        finally:
            for k, v in saved.items():
                backend.chosen.pop(k, None)
                if v is not None:
                    backend.chosen[k] = v


def test_a_shape_of_many_rows_is_measured_in_the_third_step_that_meets_it(ops):
    """Prompt portions: only a shape that comes step after step is timed (against ``torch.mm``, which stays
    unless one of the library's algorithms is clearly faster); the product is the same product either way."""
    from nanohybrid_vlm_amd.native.ops import RULE
    backend = ops.backend()
    M, N, K = 200, 384, 512
    x = rnd(M, K, dtype=torch.bfloat16, seed=61)
    w = rnd(N, K, dtype=torch.bfloat16, seed=62, scale=K ** -0.5)
    ref = x.double() @ w.double().T
    key = (M, N, K, False, False)
    saved = backend.chosen.pop(key, None), backend._met.pop(key, None)
    try:
        for step in range(3):
            backend.step_number += 1
            for _ in range(4):                               # layers of one step count once
                torch.testing.assert_close(ops.linear(x, w).double(), ref, **tol(torch.bfloat16))
            assert (key in backend.chosen) == (step == 2)
        assert backend.chosen[key] == RULE or backend.chosen[key] >= 0
        _, count = backend._library_plan(M, N, K, False)
        for how in [RULE] + list(range(min(count, 3))):
            backend.chosen[key] = how
            torch.testing.assert_close(ops.linear(x, w).double(), ref, **tol(torch.bfloat16))
    finally:
        backend.chosen.pop(key, None)
        backend._met.pop(key, None)
        if saved[0] is not None:
            backend.chosen[key] = saved[0]
        if saved[1] is not None:
            backend._met[key] = saved[1]


def test_library_products_refuse_what_they_cannot_do(ops):
    """The wrapper of the vendor's matrix library names what is wrong: an algorithm the plan does not have, a
    workspace smaller than the plan's, a plan that was never made."""
    import ctypes
    from nanohybrid_vlm_amd.native.ops import KernelError
    backend = ops.backend()
    plan, count = backend._library_plan(8, 256, 512, False)
    assert count > 0 and backend._library_plan(8, 256, 512, False) == (plan, count)      # a shape has one plan
    x = rnd(8, 512, dtype=torch.bfloat16, seed=71)
    w = rnd(256, 512, dtype=torch.bfloat16, seed=72)
    out = torch.empty(8, 256, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(KernelError, match="algorithms"):
        backend._library_product(x, w, out, count)
    ptr = lambda t: ctypes.c_void_p(t.data_ptr())
    with pytest.raises(KernelError, match="no plan"):
        backend._call("nhv_library_gemm", 10 ** 6, 0, ptr(x), ptr(w), ptr(out), None, ctypes.c_size_t(0), None, lib=backend.blas_lib())
    with pytest.raises(KernelError, match="result type"):
        backend._call("nhv_library_gemm_plan", 8, 256, 512, 7, 4, ctypes.c_size_t(0), ctypes.byref(ctypes.c_int()),
                      ctypes.byref(ctypes.c_int()), lib=backend.blas_lib())
    backend._library_product(x, w, out, 0)
    torch.testing.assert_close(out.double(), x.double() @ w.double().T, **tol(torch.bfloat16))


# ---------------------------------------------------------------- sizes drawn at random (seeded)
# The kernels choose waves, loads in flight, tiles a block and split lengths from the sizes by rules; these cases walk
# over the rules' borders at sizes nobody picked by hand.

def _random_product_sizes(seed, count, max_rows):
    import random
    rnd_ = random.Random(seed)
    sizes = []
    while len(sizes) < count:
        M = rnd_.randint(1, max_rows)
        N = rnd_.choice([rnd_.randint(1, 600), rnd_.randint(600, 9000), rnd_.randint(9000, 40000)])
        K = 8 * rnd_.choice([rnd_.randint(1, 64), rnd_.randint(64, 1000), rnd_.randint(1000, 3300)])
        if N * K <= 48_000_000:
            sizes.append((M, N, K))
    return sizes


@pytest.mark.parametrize("M,N,K", _random_product_sizes(1, 40, 16) + _random_product_sizes(2, 12, 64))
def test_products_of_few_rows_at_random_sizes(ops, M, N, K):
    x = rnd(M, K, dtype=torch.bfloat16, seed=44)
    w = rnd(N, K, dtype=torch.bfloat16, seed=45, scale=K ** -0.5)
    ref = x.double() @ w.double().T
    backend = ops.backend()
    backend.own_kernels_only = True                          # the own kernels, whatever a measurement would choose
    try:
        got = ops.linear(x, w, out_dtype=torch.float32)
        torch.testing.assert_close(got.double(), ref, rtol=1e-4, atol=2e-4)
        assert torch.equal(got, ops.linear(x, w, out_dtype=torch.float32))
        torch.testing.assert_close(ops.linear(x, w).double(), ref, **tol(torch.bfloat16))
        if N % 2 == 0:
            g, u = ref[:, :N // 2], ref[:, N // 2:]
            torch.testing.assert_close(ops.gated_linear(x, w).double(), g * torch.sigmoid(g) * u, **tol(torch.bfloat16))
    finally:
        backend.own_kernels_only = False


def _random_attention_cases(seed, count):
    import random
    rnd_ = random.Random(seed)
    cases = []
    for _ in range(count):
        Hkv = rnd_.choice([1, 2, 3, 8])
        G = rnd_.choice([1, 2, 3, 4, 5, 8, 16])
        D = 16 * rnd_.randint(1, 8) if rnd_.random() < 0.8 else 256
        page = rnd_.choice([3, 8, 16, 48, 64, 256])
        window = rnd_.choice([None, None, rnd_.randint(1, 40), rnd_.randint(41, 900)])
        cases.append((Hkv * G, Hkv, D, page, window, rnd_.randint(0, 10 ** 6)))
    return cases


@pytest.mark.parametrize("Hq,Hkv,D,page,window,seed", _random_attention_cases(3, 16))
def test_attention_kernels_at_random_sizes(ops, Hq, Hkv, D, page, window, seed):
    """Both bfloat16 attention kernels (single tokens; portions beside single tokens) at head counts, group sizes,
    head sizes, page sizes, windows and lengths drawn at random."""
    import random
    rnd_ = random.Random(seed)
    scale = D ** -0.5
    # single tokens: the split-key kernel
    lens = [rnd_.choice([rnd_.randint(1, 70), rnd_.randint(70, 700), rnd_.randint(700, 2600)]) for _ in range(rnd_.randint(1, 9))]
    q_lens = [1] * len(lens)
    q, kc, vc, batch, bt, ks, vs, qs = _paged_setup(torch.bfloat16, lens, q_lens, Hq, Hkv, D, page, seed=seed, scale=1.5)
    out = ops.paged_attention(q, kc, vc, batch, bt, scale, window)
    torch.testing.assert_close(out.double().cpu(), _attention_reference(qs, ks, vs, lens, q_lens, scale, window),
                               **tol(torch.bfloat16))
    # portions with and without earlier keys beside single tokens: the matrix-core kernel for prompts
    lens = [rnd_.randint(1, 1200) for _ in range(rnd_.randint(1, 5))]
    q_lens = [rnd_.choice([1, n, rnd_.randint(1, n)]) for n in lens]
    q_lens[0] = max(2, min(lens[0], q_lens[0])) if lens[0] > 1 else 1
    if max(q_lens) == 1:
        lens.append(300)
        q_lens.append(77)
    q, kc, vc, batch, bt, ks, vs, qs = _paged_setup(torch.bfloat16, lens, q_lens, Hq, Hkv, D, page, seed=seed + 1, scale=1.5)
    out = ops.paged_attention(q, kc, vc, batch, bt, scale, window)
    torch.testing.assert_close(out.double().cpu(), _attention_reference(qs, ks, vs, lens, q_lens, scale, window),
                               **tol(torch.bfloat16))

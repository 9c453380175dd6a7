"""The entry point that allocates nothing: ``nhv_decode_attention_bf16_no_alloc`` keeps the splits' partial results
in an array of the library's own device image instead of taking scratch tensors from the caller. Called through
``ctypes`` as a caller outside the package would; its output is bit for bit that of ``nhv_decode_attention_bf16``
on two calls in a row, the second with a smaller input (the array still holds the first call's results then)."""
import ctypes

import pytest
import torch

from test_kernels_gpu import _attention_reference, _paged_setup, tol

pytestmark = pytest.mark.gpu


def _library(head_dim):
    from nanohybrid_vlm_amd.native import library, ops
    path = library.build_library(f"nhv_attention_d{head_dim}", ops.ATTENTION_SOURCES, [f"-DNHV_HEAD_DIM={head_dim}"])
    lib = ctypes.CDLL(path)
    lib.nhv_last_error.restype = ctypes.c_char_p
    lib.nhv_decode_attention_no_alloc_limit.restype = ctypes.c_size_t
    return lib


def _p(t):
    return ctypes.c_void_p(t.data_ptr())


def _both_ways(lib, lens, Hq, Hkv, D, page, split_len, seed, window=0):
    q, kc, vc, batch, bt, ks, vs, qs = _paged_setup(torch.bfloat16, lens, [1] * len(lens), Hq, Hkv, D, page, seed=seed, scale=1.5)
    T = len(lens)
    n_splits = -(-max(lens) // split_len)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    scale = ctypes.c_float(D ** -0.5)
    # the existing entry point, with scratch tensors of the caller
    part_o = torch.full((T, Hq, n_splits, D), float("nan"), dtype=torch.float32, device="cuda")
    part_ml = torch.full((T, Hq, n_splits, 2), float("nan"), dtype=torch.float32, device="cuda")
    want = torch.empty_like(q)
    rc = lib.nhv_decode_attention_bf16(_p(q), _p(kc), _p(vc), _p(want), _p(part_o), _p(part_ml), _p(batch.token_req),
                                       _p(batch.positions), _p(bt), bt.shape[1], T, Hq, Hkv, page, scale, window, split_len,
                                       n_splits, stream)
    assert rc == 0, lib.nhv_last_error().decode()
    # the new one: inputs and the output only
    got = torch.full_like(q, float("nan"))
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats()["allocation.all.allocated"], torch.cuda.mem_get_info()[0]
    rc = lib.nhv_decode_attention_bf16_no_alloc(_p(q), _p(kc), _p(vc), _p(got), _p(batch.token_req), _p(batch.positions),
                                                _p(bt), bt.shape[1], T, Hq, Hkv, page, scale, window, split_len, n_splits,
                                                stream)
    assert rc == 0, lib.nhv_last_error().decode()
    torch.cuda.synchronize()
    assert torch.cuda.memory_stats()["allocation.all.allocated"] == before[0]
    free_after = torch.cuda.mem_get_info()[0]
    assert torch.equal(got, want), f"differs from the existing entry point by {(got.float() - want.float()).abs().max().item():.3e}"
    ref = _attention_reference(qs, ks, vs, lens, [1] * len(lens), D ** -0.5, window)
    torch.testing.assert_close(got.double().cpu(), ref, **tol(torch.bfloat16))
    return before[1], free_after


@pytest.mark.parametrize("Hq,Hkv,D,page", [(8, 2, 128, 256), (6, 1, 48, 16)])
def test_no_alloc_entry_point_equals_the_existing_one(Hq, Hkv, D, page):
    lib = _library(D)
    assert lib.nhv_decode_attention_no_alloc_limit() == 4 << 20
    # first call (its first use on this device asks for the array's address)
    _both_ways(lib, [3000, 17, 1025, 64, 2049, 500], Hq, Hkv, D, page, split_len=64, seed=5)
    # second call, smaller in every way: fewer tokens, shorter contexts, longer splits; the array still holds the
    # first call's partial results, none of which may leak into this one
    before, after = _both_ways(lib, [300, 5], Hq, Hkv, D, page, split_len=128, seed=6)
    assert before == after, "the device's free memory changed over the call"
    # and a third with a window
    before, after = _both_ways(lib, [700, 90, 33], Hq, Hkv, D, page, split_len=64, seed=7, window=100)
    assert before == after, "the device's free memory changed over the call"


def test_no_alloc_entry_point_refuses_what_does_not_fit():
    lib = _library(128)
    lens = [4000] * 8
    q, kc, vc, batch, bt, *_ = _paged_setup(torch.bfloat16, lens, [1] * 8, 32, 8, 128, 256, seed=1)
    out = torch.zeros_like(q)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    # 8 tokens x 32 heads x 63 splits x 130 floats = 8.4 MB: beyond the 4 MiB the library holds
    rc = lib.nhv_decode_attention_bf16_no_alloc(_p(q), _p(kc), _p(vc), _p(out), _p(batch.token_req), _p(batch.positions),
                                                _p(bt), bt.shape[1], 8, 32, 8, 256, ctypes.c_float(0.088), 0, 64, 63, stream)
    assert rc == 1
    message = lib.nhv_last_error().decode()
    assert "scratch" in message and "8386560" in message and str(4 << 20) in message
    torch.cuda.synchronize()
    assert not out.any(), "a refused call launches nothing"
    # the same call with splits of 256 keys fits (16 splits: 2.1 MB)
    rc = lib.nhv_decode_attention_bf16_no_alloc(_p(q), _p(kc), _p(vc), _p(out), _p(batch.token_req), _p(batch.positions),
                                                _p(bt), bt.shape[1], 8, 32, 8, 256, ctypes.c_float(0.088), 0, 256, 16, stream)
    assert rc == 0, lib.nhv_last_error().decode()
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all() and out.any()


def test_no_alloc_entry_point_recorded_into_a_graph():
    """After the address of the array is known on the device (``nhv_decode_attention_no_alloc_init``, outside any
    capture) a call only launches kernels: it is recorded into a HIP graph and replayed, with other work between
    the replays and with other inputs in the same buffers, and gives the existing entry point's result each time."""
    Hq, Hkv, D, page, split_len = 8, 2, 128, 64, 128
    lib = _library(D)
    assert lib.nhv_decode_attention_no_alloc_init() == 0, lib.nhv_last_error().decode()
    lens = [900, 130, 64, 513]
    q, kc, vc, batch, bt, ks, vs, qs = _paged_setup(torch.bfloat16, lens, [1] * len(lens), Hq, Hkv, D, page, seed=11, scale=1.5)
    T, n_splits = len(lens), -(-max(lens) // split_len)
    scale = ctypes.c_float(D ** -0.5)
    got = torch.zeros_like(q)
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    with torch.cuda.graph(graph, stream=side):
        rc = lib.nhv_decode_attention_bf16_no_alloc(_p(q), _p(kc), _p(vc), _p(got), _p(batch.token_req), _p(batch.positions),
                                                    _p(bt), bt.shape[1], T, Hq, Hkv, page, scale, 0, split_len, n_splits,
                                                    ctypes.c_void_p(side.cuda_stream))
    assert rc == 0, lib.nhv_last_error().decode()
    part_o = torch.empty((T, Hq, n_splits, D), dtype=torch.float32, device="cuda")
    part_ml = torch.empty((T, Hq, n_splits, 2), dtype=torch.float32, device="cuda")
    for replay in range(3):
        if replay:
            q.copy_(torch.randn_like(q.float()).to(q.dtype))          # other queries in the same buffer
        want = torch.empty_like(q)
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        rc = lib.nhv_decode_attention_bf16(_p(q), _p(kc), _p(vc), _p(want), _p(part_o), _p(part_ml), _p(batch.token_req),
                                           _p(batch.positions), _p(bt), bt.shape[1], T, Hq, Hkv, page, scale, 0, split_len,
                                           n_splits, stream)
        assert rc == 0, lib.nhv_last_error().decode()
        got.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"replay {replay}"

"""The decode-attention entry point that allocates nothing (csrc/no_alloc.h), called through ctypes:
its output must equal the workspace-taking entry point's bit for bit, on two calls in a row (the
second with a smaller input, so that the scratch array still holds the first call's partial
results), and a call that needs more scratch than the array has must be refused."""
import ctypes

import pytest
import torch

from gpu_util import DEV, paged_cache, table_tensor

pytestmark = pytest.mark.gpu


def _ptr(t):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _problem(seed, nq, nkv, hd, P, lens):
    g = torch.Generator().manual_seed(seed)
    rnd = lambda *s: torch.randn(*s, generator=g).to(torch.bfloat16).float()   # noqa: E731
    ks = [rnd(S, nkv, hd) for S in lens]
    vs = [rnd(S, nkv, hd) for S in lens]
    k_pool, v_pool, tables = paged_cache(ks, vs, P, torch.bfloat16, DEV, seed=seed)
    q = rnd(len(lens), nq * hd).to(DEV, torch.bfloat16)
    positions = torch.tensor([S - 1 for S in lens], dtype=torch.int32, device=DEV)
    entry = torch.arange(len(lens), dtype=torch.int32, device=DEV)
    return q, k_pool, v_pool, positions, entry, table_tensor(tables, DEV)


def _call(lib, static, q, k_pool, v_pool, positions, entry, bt, P, nq, nkv, hd, splits, waves):
    n = q.shape[0]
    out = torch.full_like(q, float("nan"))
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    head = (_ptr(q), ctypes.c_int(q.stride(0)), _ptr(out), ctypes.c_int(out.stride(0)), _ptr(k_pool), _ptr(v_pool),
            _ptr(None), ctypes.c_int(n), _ptr(positions), _ptr(entry), _ptr(bt), ctypes.c_int(bt.stride(0)),
            ctypes.c_int(P), ctypes.c_int(nq), ctypes.c_int(nkv), ctypes.c_int(hd), ctypes.c_float(hd ** -0.5),
            ctypes.c_int(0), ctypes.c_int(splits), ctypes.c_int(waves))
    if static:
        rc = lib.ullm_attention_decode_static(*head, stream)
    else:
        lib.ullm_attention_decode_workspace.restype = ctypes.c_longlong
        need = lib.ullm_attention_decode_workspace(ctypes.c_int(n), ctypes.c_int(nq), ctypes.c_int(hd), ctypes.c_int(splits))
        ws = torch.empty(max(1, need), dtype=torch.float32, device=DEV)
        rc = lib.ullm_attention_decode(*head, _ptr(ws), stream)
    torch.cuda.synchronize()
    return rc, out


def test_decode_attention_without_allocation_equals_the_workspace_entry_point():
    from ullm_amd.kernels import build
    lib = build.load("attention_mfma")
    lib.ullm_attention_decode_static_capacity.restype = ctypes.c_longlong
    capacity = lib.ullm_attention_decode_static_capacity()
    assert capacity == 2 * 1024 * 1024
    nq, nkv, hd, P = 32, 8, 128, 16
    # first a batch of four long requests cut seven ways, then a smaller one cut three ways: the second
    # call finds the first call's partial results in the scratch array and must not be disturbed by them
    for seed, lens, splits, waves in ((1, [700, 1153, 90, 333], 7, 8), (2, [130, 45], 3, 4), (3, [64], 1, 4)):
        args = _problem(seed, nq, nkv, hd, P, lens)
        rc_ws, want = _call(lib, False, *args, P, nq, nkv, hd, splits, waves)
        rc_st, got = _call(lib, True, *args, P, nq, nkv, hd, splits, waves)
        assert rc_ws == 0 and rc_st == 0
        assert not torch.isnan(got).any()
        assert torch.equal(got, want), (seed, (got.float() - want.float()).abs().max())
    # beyond the array: refused, nothing launched (the output keeps its fill)
    lens = [40] * 64
    args = _problem(4, nq, nkv, hd, P, lens)
    splits = capacity // (len(lens) * nq * (hd + 4)) + 1
    rc, out = _call(lib, True, *args, P, nq, nkv, hd, splits, 4)
    assert rc == -4
    assert torch.isnan(out).all()


def test_decode_attention_without_allocation_under_graph_capture():
    """After one call outside capture (the capacity query looks the array up), the entry point is captured
    into a HIP graph and replayed with other inputs in the same tensors, eager work between the replays; every
    replay equals the workspace entry point run eagerly, and the call allocates no device memory."""
    from ullm_amd.kernels import build
    lib = build.load("attention_mfma")
    lib.ullm_attention_decode_static_capacity.restype = ctypes.c_longlong
    assert lib.ullm_attention_decode_static_capacity() > 0          # warm-up on this device, outside capture
    nq, nkv, hd, P, splits, waves = 32, 8, 128, 16, 5, 4
    lens = [300, 47, 1025]
    q, k_pool, v_pool, positions, entry, bt = _problem(7, nq, nkv, hd, P, lens)
    out = torch.full_like(q, float("nan"))

    def launch(stream):
        return lib.ullm_attention_decode_static(
            _ptr(q), ctypes.c_int(q.stride(0)), _ptr(out), ctypes.c_int(out.stride(0)), _ptr(k_pool), _ptr(v_pool),
            _ptr(None), ctypes.c_int(len(lens)), _ptr(positions), _ptr(entry), _ptr(bt), ctypes.c_int(bt.stride(0)),
            ctypes.c_int(P), ctypes.c_int(nq), ctypes.c_int(nkv), ctypes.c_int(hd), ctypes.c_float(hd ** -0.5),
            ctypes.c_int(0), ctypes.c_int(splits), ctypes.c_int(waves), ctypes.c_void_p(stream.cuda_stream))
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    assert launch(torch.cuda.current_stream()) == 0
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before                  # torch's allocator was not asked for anything
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        assert launch(torch.cuda.current_stream()) == 0
    for seed in (8, 9, 10):
        # other numbers in the same tensors (rows of the pools that no request holds stay as they are)
        q.copy_(torch.randn(q.shape, generator=torch.Generator().manual_seed(seed)).to(q.dtype))
        k_pool.neg_()
        v_pool.mul_(0.5)
        out.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        rc, want = _call(lib, False, q, k_pool, v_pool, positions, entry, bt, P, nq, nkv, hd, splits, waves)
        assert rc == 0 and torch.equal(out, want), seed

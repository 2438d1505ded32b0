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

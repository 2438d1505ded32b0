"""Each HIP kernel alone against its plain reference, at sizes other than the engine's tests use."""
import math

import pytest
import torch
import torch.nn.functional as F

import plain_qwen3 as plain
from gpu_util import DEV, paged_cache, table_tensor, tol

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(scope="module")
def ops():
    from ullm_amd.kernels import ops as o
    return o


def test_feed_tokens(ops):
    """Token ids a step takes from the sampler's output of the step before: only where the map says so."""
    ids = torch.tensor([5, 0, 9, 0, 0, 7], dtype=torch.int32, device=DEV)
    feed = torch.tensor([-1, 2, -1, 0, 3, -1], dtype=torch.int32, device=DEV)
    source = torch.tensor([40, 41, 42, 43], dtype=torch.int32, device=DEV)
    ops.feed_tokens(ids, feed, source)
    assert ids.tolist() == [5, 42, 9, 40, 43, 7]
    big = torch.arange(1000, dtype=torch.int32, device=DEV)
    feed = torch.full((1000,), -1, dtype=torch.int32, device=DEV)
    feed[::3] = torch.arange(334, dtype=torch.int32, device=DEV) % 4
    want = big.clone()
    want[::3] = source[(torch.arange(334, device=DEV) % 4).long()]
    ops.feed_tokens(big, feed, source)
    assert torch.equal(big, want)
    # an index past the source leaves the id alone (the host never packs one)
    ids = torch.tensor([1, 2], dtype=torch.int32, device=DEV)
    ops.feed_tokens(ids, torch.tensor([9, -1], dtype=torch.int32, device=DEV), source)
    assert ids.tolist() == [1, 2]


@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding(ops, dtype):
    torch.manual_seed(0)
    table = torch.randn(1003, 200).to(DEV, dtype)
    ids = torch.tensor([0, 1002, 17, 17, 500], dtype=torch.int32, device=DEV)
    out = ops.embedding(ids, table)
    assert out.dtype == torch.float32 and torch.equal(out, table.float()[ids.long()])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H", [48, 1000, 5120])
def test_add_rmsnorm(ops, dtype, H):
    torch.manual_seed(1)
    T, eps = 7, 1e-5
    res = torch.randn(T, H, device=DEV) * 3
    branch = torch.randn(T, H, device=DEV).to(dtype)
    gain = (1 + 0.1 * torch.randn(H, device=DEV))
    s = res + branch.float()
    want = plain.rms_norm(s.cpu(), gain.cpu(), eps)
    res_in = res.clone()
    y = ops.add_rmsnorm(branch, res_in, gain, eps, dtype)
    assert torch.equal(res_in, s)                                    # the stream is the unrounded 32-bit sum
    assert (y.float().cpu() - want).abs().max() <= tol(dtype, want)
    # rows: only the chosen rows, the stream untouched
    rows = torch.tensor([6, 2, 2], dtype=torch.int32, device=DEV)
    res_in = res.clone()
    y = ops.add_rmsnorm(branch, res_in, gain, eps, dtype, rows=rows)
    assert torch.equal(res_in, res)
    assert (y.float().cpu() - want[[6, 2, 2]]).abs().max() <= tol(dtype, want)
    # no branch: plain norm, equals the library routine
    y = ops.add_rmsnorm(None, res.clone(), gain, eps, torch.float32)
    assert torch.allclose(y, F.rms_norm(res, (H,), gain, eps), atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize("dtype", DTYPES)
def test_silu_mul(ops, dtype):
    torch.manual_seed(2)
    gu = (torch.randn(5, 2 * 333, device=DEV) * 2).to(dtype)
    want = plain.silu_and_mul(gu.float().cpu())
    got = ops.silu_mul(gu)
    assert (got.float().cpu() - want).abs().max() <= tol(dtype, want)
    gu[:, :333] = 0
    assert torch.all(ops.silu_mul(gu) == 0)


@pytest.mark.parametrize("dtype", DTYPES)
def test_add_bias(ops, dtype):
    """The bias of a library product is added by a kernel of our own, in 32-bit, in place, also into a view."""
    torch.manual_seed(3)
    y = (torch.randn(37, 203, device=DEV) * 3).to(dtype)
    bias = torch.randn(203, device=DEV)
    want = (y.float() + bias).to(dtype)
    assert ops.add_bias(y, bias) is y and torch.equal(y, want)
    wide = (torch.randn(5, 64, device=DEV)).to(dtype)
    keep = wide.clone()
    ops.add_bias(wide[:, 8:40], bias[:32].contiguous())
    assert torch.equal(wide[:, 8:40], (keep[:, 8:40].float() + bias[:32]).to(dtype))
    assert torch.equal(wide[:, :8], keep[:, :8]) and torch.equal(wide[:, 40:], keep[:, 40:])
    # through the dispatch: a biased bfloat16 product with more rows than the weight-streaming kernel takes
    if dtype == torch.bfloat16:
        a, w = torch.randn(40, 64, device=DEV).to(dtype), torch.randn(96, 64, device=DEV).to(dtype)
        b = torch.randn(96, device=DEV)
        for out_dtype in (torch.bfloat16, torch.float32):
            got = ops.gemm_bf16(a, w, b, out_dtype=out_dtype)
            ref = a.float() @ w.float().T + b
            assert got.dtype == out_dtype and (got.float() - ref).abs().max() <= tol(dtype, ref)


@pytest.mark.parametrize("shape", [(1, 50, 70), (5, 129, 33), (70, 64, 16), (3, 503, 96)])
def test_gemm_simple(ops, shape):
    torch.manual_seed(3)
    M, N, K = shape
    a, w, b = torch.randn(M, K, device=DEV), torch.randn(N, K, device=DEV), torch.randn(N, device=DEV)
    want = (a.double() @ w.double().T + b.double()).float()
    got = ops.gemm_simple(a, w, b)
    assert (got - want).abs().max() <= 2e-5 * want.abs().max()
    # a row's result does not depend on the other rows (bitwise)
    assert torch.equal(ops.gemm_simple(a[:1].contiguous(), w, b), got[:1])
    ab, wb = a.bfloat16(), w.bfloat16()
    want = ab.double() @ wb.double().T
    got = ops.gemm_simple(ab, wb, out_dtype=torch.float32)
    assert got.dtype == torch.float32 and (got - want.float()).abs().max() <= 2e-5 * want.abs().max()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("cfg", [dict(nq=6, nkv=2, hd=48, P=8, rot=48, style=1, norm=True),
                                 dict(nq=5, nkv=5, hd=64, P=16, rot=32, style=1, norm=True),
                                 dict(nq=4, nkv=1, hd=16, P=4, rot=16, style=2, norm=False),
                                 dict(nq=2, nkv=2, hd=256, P=32, rot=0, style=0, norm=True),
                                 dict(nq=8, nkv=2, hd=128, P=16, rot=128, style=1, norm=True),     # 16 lanes a head
                                 dict(nq=5, nkv=1, hd=128, P=16, rot=64, style=2, norm=True),
                                 dict(nq=3, nkv=3, hd=32, P=8, rot=16, style=1, norm=False),       # 4 lanes a head
                                 dict(nq=70, nkv=2, hd=32, P=8, rot=32, style=2, norm=True),       # heads beyond one block
                                 dict(nq=2, nkv=1, hd=512, P=16, rot=512, style=1, norm=True),     # a whole wave a head
                                 dict(nq=4, nkv=2, hd=64, P=16, rot=24, style=1, norm=True)])      # rot no multiple of 16
def test_qk_norm_rope_write(ops, dtype, cfg):
    torch.manual_seed(4)
    nq, nkv, hd, P, rot, style = (cfg[k] for k in ("nq", "nkv", "hd", "P", "rot", "style"))
    eps, theta = 1e-5, 5000.0
    # two entries: positions 9..14 of request 0 and position 40 of request 1
    positions = torch.tensor([9, 10, 11, 12, 13, 14, 40], dtype=torch.int32)
    entry = torch.tensor([0, 0, 0, 0, 0, 0, 1], dtype=torch.int32)
    T = positions.numel()
    need = [14 // P + 1, 40 // P + 1]
    ids = torch.randperm(sum(need) + 2).tolist()               # page ids in no order
    tables = [ids[:need[0]], ids[need[0]:need[0] + need[1]]]
    n_pages = len(ids)
    bt = table_tensor(tables, DEV)
    qkv = torch.randn(T, (nq + 2 * nkv) * hd).to(dtype)
    qg, kg = 1 + 0.2 * torch.randn(hd), 1 + 0.2 * torch.randn(hd)
    k_pool = torch.zeros(n_pages, nkv, P, hd, dtype=dtype, device=DEV)
    v_pool = torch.zeros(n_pages, nkv, hd, P, dtype=dtype, device=DEV)
    q_out = torch.empty(T, nq * hd, dtype=dtype, device=DEV)
    table = None
    if style:
        inv = 1.0 / (theta ** (torch.arange(0, rot, 2, dtype=torch.float32) / rot))
        ang = torch.arange(64, dtype=torch.float32)[:, None] * inv[None]
        table = torch.cat((ang.cos(), ang.sin()), -1).contiguous().to(DEV)
    ops.qk_norm_rope_write(qkv.to(DEV), q_out, qg.to(DEV) if cfg["norm"] else None, kg.to(DEV) if cfg["norm"] else None,
                           eps, table, rot, style, positions.to(DEV), entry.to(DEV), bt, k_pool, v_pool, P, nq, nkv,
                           hd, write_kv=True)
    x = qkv.float()
    q, k, v = x[:, :nq * hd].view(T, nq, hd), x[:, nq * hd:(nq + nkv) * hd].view(T, nkv, hd), x[:, (nq + nkv) * hd:].view(T, nkv, hd)
    if cfg["norm"]:
        q, k = plain.rms_norm(q, qg, eps), plain.rms_norm(k, kg, eps)
    if style:
        cos, sin = plain.rope_cos_sin(positions, rot, theta)

        def rotate(t):
            r, rest = t[..., :rot], t[..., rot:]
            if style == 1:
                r = plain.apply_rope_concat_layout(r, cos, sin)
            else:       # adjacent pairs (2i, 2i+1)
                a, b = r[..., 0::2], r[..., 1::2]
                c, s = cos.unsqueeze(1), sin.unsqueeze(1)
                r = torch.stack((a * c - b * s, b * c + a * s), -1).flatten(-2)
            return torch.cat((r, rest), -1)
        q, k = rotate(q), rotate(k)
    assert (q_out.float().cpu().view(T, nq, hd) - q).abs().max() <= tol(dtype, q)
    for t in range(T):
        pos, e = int(positions[t]), int(entry[t])
        page, row = tables[e][pos // P], pos % P
        assert (k_pool[page, :, row].float().cpu() - k[t]).abs().max() <= tol(dtype, k)
        assert torch.equal(v_pool[page, :, :, row].float().cpu(), v[t])
    written = sum(1 for _ in range(T))
    assert int((k_pool.float().abs().sum(-1) > 0).sum()) == written * nkv       # nothing else was touched


def test_stacks_of_partial_sums_added_to_one_result(ops, monkeypatch):
    """A first projection above the rows of the weight-streaming kernels, where the table says so: the partial
    sums of slices of the inner dimension, added in order by a kernel of its own, with the bias, rounded once."""
    import dataclasses
    from ullm_amd.kernels import dispatch
    torch.manual_seed(12)
    for S, M, N in ((5, 70, 36), (1, 3, 4), (8, 256, 1024)):
        stacks = torch.randn(S, M, N, device=DEV)
        bias = torch.randn(N, device=DEV)
        want = stacks[0].clone()
        for s in range(1, S):
            want += stacks[s]
        assert torch.equal(ops.sum_stacks(stacks, out_dtype=torch.float32), want)
        assert torch.equal(ops.sum_stacks(stacks, bias), (want + bias).to(torch.bfloat16))
    rules = dispatch.default_limits
    monkeypatch.setattr(dispatch, "_table", {})
    monkeypatch.setattr(dispatch, "default_limits", lambda c, k: dataclasses.replace(rules(c, k), sums_from=65, sums_to=256))
    for M, N, K in ((96, 1536, 1024), (200, 520, 2048), (65, 6144, 4096)):
        x, w = torch.randn(M, K, device=DEV).bfloat16(), (torch.randn(N, K, device=DEV) * 0.05).bfloat16()
        bias = torch.randn(N, device=DEV)
        calls = []
        real = ops.sum_stacks
        monkeypatch.setattr(ops, "sum_stacks", lambda *a, **k: (calls.append(1), real(*a, **k))[1])
        got = ops.gemm_bf16(x, w, bias)
        monkeypatch.setattr(ops, "sum_stacks", real)
        assert calls, "the projection did not take the partial sums"
        want = x.float() @ w.float().t() + bias
        assert got.dtype == torch.bfloat16 and (got.float() - want).abs().max() <= tol(torch.bfloat16, want)
        # a row's result does not depend on the other rows
        assert torch.equal(ops.gemm_bf16(x[:70].contiguous(), w, bias)[:65], got[:65])
    monkeypatch.setattr(dispatch, "_table", None)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("cfg", [dict(nq=32, nkv=8, hd=128, P=16, rot=128, style=1),    # 48 heads: three in turn per thread
                                 dict(nq=70, nkv=2, hd=32, P=8, rot=32, style=2),       # 74 heads of 4 lanes: two in turn
                                 dict(nq=5, nkv=1, hd=128, P=16, rot=64, style=2),      # 7 heads: one block, one turn
                                 dict(nq=40, nkv=40, hd=64, P=16, rot=32, style=1)])    # 120 heads: four in turn, a spare turn
def test_qk_norm_rope_write_of_a_long_prompt(ops, dtype, cfg):
    """From 1 024 tokens on a thread takes several heads in turn with one fetch of its cosines and sines; what it
    writes is, bit for bit, what the same tokens give in portions below that length (which the test above
    checks against the plain formulas)."""
    torch.manual_seed(41)
    nq, nkv, hd, P, rot, style = (cfg[k] for k in ("nq", "nkv", "hd", "P", "rot", "style"))
    T = 1100
    positions = torch.arange(T, dtype=torch.int32, device=DEV)
    entry = torch.zeros(T, dtype=torch.int32, device=DEV)
    n_pages = -(-T // P)
    bt = table_tensor([torch.randperm(n_pages).tolist()], DEV)
    qkv = torch.randn(T, (nq + 2 * nkv) * hd).to(dtype).to(DEV)
    qg, kg = (1 + 0.2 * torch.randn(hd)).to(DEV), (1 + 0.2 * torch.randn(hd)).to(DEV)
    inv = 1.0 / (10000.0 ** (torch.arange(0, rot, 2, dtype=torch.float32) / rot))
    ang = torch.arange(T + 5, dtype=torch.float32)[:, None] * inv[None]
    table = torch.cat((ang.cos(), ang.sin()), -1).contiguous().to(DEV)
    results = []
    for portions in ([T], [500, 400, 200]):
        k_pool = torch.zeros(n_pages, nkv, P, hd, dtype=dtype, device=DEV)
        v_pool = torch.zeros(n_pages, nkv, hd, P, dtype=dtype, device=DEV)
        q_out = torch.zeros(T, nq * hd, dtype=dtype, device=DEV)
        at = 0
        for n in portions:
            ops.qk_norm_rope_write(qkv[at:at + n], q_out[at:at + n], qg, kg, 1e-6, table, rot, style, positions[at:at + n],
                                   entry[at:at + n], bt, k_pool, v_pool, P, nq, nkv, hd, write_kv=True)
            at += n
        results.append((q_out, k_pool, v_pool))
    for whole, cut in zip(*results):
        assert torch.equal(whole, cut)
    assert float(results[0][0].float().abs().sum()) > 0 and float(results[0][1].float().abs().sum()) > 0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("cfg", [dict(nq=8, nkv=2, hd=128, P=16), dict(nq=4, nkv=4, hd=64, P=8),
                                 dict(nq=2, nkv=1, hd=256, P=32), dict(nq=4, nkv=2, hd=32, P=24),
                                 dict(nq=4, nkv=2, hd=64, P=12),      # pages that do not hold whole groups of 8
                                 dict(nq=2, nkv=2, hd=512, P=16)])    # too wide for the blocks that write runs
def test_cache_write_of_many_tokens(ops, dtype, cfg):
    """With many tokens in the batch the values are written in runs of eight positions: portions that
    start at odd positions, at 0, single tokens between them, an entry without pages, and a
    portion that ends in the middle of a group all land where the token-by-token write puts them."""
    torch.manual_seed(14)
    nq, nkv, hd, P = (cfg[k] for k in ("nq", "nkv", "hd", "P"))
    # (entry, first position, tokens); entry 3 has no pages (a padding entry of a captured batch)
    portions = [(0, 77, 1), (1, 5, 146), (2, 0, 100), (3, 9, 1), (4, 300, 1), (5, 64, 43), (3, 10, 1), (6, 8, 8)]
    positions = torch.cat([torch.arange(f, f + n) for _, f, n in portions]).int()
    entry = torch.cat([torch.full((n,), e) for e, _, n in portions]).int()
    T = positions.numel()
    assert T >= 128
    last = {}
    for e, f, n in portions:
        last[e] = max(last.get(e, 0), f + n - 1)
    need = {e: (0 if e == 3 else last[e] // P + 1) for e in last}
    ids = torch.randperm(sum(need.values()) + 3).tolist()
    tables, at = [], 0
    for e in range(7):
        tables.append(ids[at:at + need[e]])
        at += need[e]
    n_pages = len(ids)
    width = max(len(t) for t in tables)
    bt = torch.full((7, width), -1, dtype=torch.int32)
    for e, t in enumerate(tables):
        bt[e, :len(t)] = torch.tensor(t, dtype=torch.int32)
    bt = bt.to(DEV)
    qkv = torch.randn(T, (nq + 2 * nkv) * hd).to(dtype)
    k_pool = torch.zeros(n_pages, nkv, P, hd, dtype=dtype, device=DEV)
    v_pool = torch.zeros(n_pages, nkv, hd, P, dtype=dtype, device=DEV)
    q_out = torch.empty(T, nq * hd, dtype=dtype, device=DEV)
    ops.qk_norm_rope_write(qkv.to(DEV), q_out, None, None, 1e-6, None, 0, 0, positions.to(DEV), entry.to(DEV), bt,
                           k_pool, v_pool, P, nq, nkv, hd, write_kv=True)
    x = qkv.float()
    k, v = x[:, nq * hd:(nq + nkv) * hd].view(T, nkv, hd), x[:, (nq + nkv) * hd:].view(T, nkv, hd)
    assert torch.equal(q_out.float().cpu(), x[:, :nq * hd])
    want_k = torch.zeros(n_pages, nkv, P, hd)
    want_v = torch.zeros(n_pages, nkv, hd, P)
    for t in range(T):
        pos, e = int(positions[t]), int(entry[t])
        if e == 3:
            continue
        want_k[tables[e][pos // P], :, pos % P] = k[t]
        want_v[tables[e][pos // P], :, :, pos % P] = v[t]
    assert torch.equal(k_pool.float().cpu(), want_k)
    assert torch.equal(v_pool.float().cpu(), want_v)


def reference_attention(qs, ks, vs, scale, window):
    """qs[b]: [n_b, nq, hd] queries at the last n_b positions of sequence b (ks[b]: [S_b, nkv, hd])."""
    outs = []
    for q, k, v in zip(qs, ks, vs):
        n, S = q.shape[0], k.shape[0]
        full_q = torch.zeros(S, q.shape[1], q.shape[2])
        full_q[S - n:] = q
        outs.append(plain.causal_gqa_attention(full_q, k, v, scale, window)[S - n:])
    return torch.cat(outs)


ATT_CASES = [dict(nq=4, nkv=2, hd=16, P=4, lens=[(5, 5), (1, 37), (7, 20)], window=0),
             dict(nq=6, nkv=2, hd=48, P=8, lens=[(1, 1), (2, 130), (33, 33), (1, 64)], window=0),
             dict(nq=8, nkv=1, hd=128, P=16, lens=[(1, 300), (1, 17), (3, 48)], window=0),
             dict(nq=3, nkv=3, hd=80, P=16, lens=[(9, 40), (1, 100)], window=11),
             dict(nq=4, nkv=2, hd=256, P=32, lens=[(1, 70), (20, 64)], window=0)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("case", ATT_CASES)
def test_paged_attention_generic(ops, dtype, case):
    torch.manual_seed(5)
    nq, nkv, hd, P, window = (case[k] for k in ("nq", "nkv", "hd", "P", "window"))
    rnd = lambda *s: torch.randn(*s).to(dtype).float()   # noqa: E731
    ks = [rnd(S, nkv, hd) for _, S in case["lens"]]
    vs = [rnd(S, nkv, hd) for _, S in case["lens"]]
    qs = [rnd(n, nq, hd) for n, _ in case["lens"]]
    k_pool, v_pool, tables = paged_cache(ks, vs, P, dtype, DEV)          # unused rows are NaN
    positions = torch.cat([torch.arange(S - n, S) for n, S in case["lens"]]).int().to(DEV)
    entry = torch.cat([torch.full((n,), b) for b, (n, _) in enumerate(case["lens"])]).int().to(DEV)
    q = torch.cat(qs).reshape(-1, nq * hd).to(DEV, dtype)
    scale = hd ** -0.5
    got = ops.paged_attention_generic(q, k_pool, v_pool, positions, entry, table_tensor(tables, DEV), P, nq, nkv,
                                      hd, scale, window)
    want = reference_attention(qs, ks, vs, scale, window).reshape(-1, nq * hd)
    assert not torch.isnan(got).any()
    assert (got.float().cpu() - want).abs().max() <= tol(dtype, want)


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_finds_one_far_key_at_every_edge(ops, dtype):
    """One key is made to dominate: the output must be its value row.  The key is placed at page edges,
    at the first and last position and at both edges of a window, for a decoded token and for the last
    token of a portion."""
    torch.manual_seed(6)
    nq, nkv, hd, P, S = 4, 2, 32, 8, 203
    for window in (0, 50):
        lo = 0 if window == 0 else S - window
        for target in sorted(t for t in {lo, lo + 1, (lo // P + 1) * P - 1, (lo // P + 1) * P, 127, 128, 167, 168,
                                        S - 2, S - 1} if t >= lo):
            for n in (1, 5):
                k = torch.randn(S, nkv, hd) * 0.1
                v = torch.randn(S, nkv, hd).to(dtype).float()
                q = torch.randn(n, nq, hd) * 0.1
                direction = torch.randn(hd)
                direction /= direction.norm()
                k[target] = 30.0 * direction
                q[-1] = 30.0 * direction                      # the last query looks at `target` only
                k, q = k.to(dtype).float(), q.to(dtype).float()
                k_pool, v_pool, tables = paged_cache([k], [v], P, dtype, DEV, seed=target)
                positions = torch.arange(S - n, S).int().to(DEV)
                entry = torch.zeros(n, dtype=torch.int32, device=DEV)
                got = ops.paged_attention_generic(q.reshape(n, -1).to(DEV, dtype), k_pool, v_pool, positions, entry,
                                                  table_tensor(tables, DEV), P, nq, nkv, hd, 1.0, window)
                got = got.float().cpu().view(n, nq, hd)[-1]
                for h in range(nq):
                    assert (got[h] - v[target, h // 2]).abs().max() < 2e-2, (window, target, n, h)
        if window:
            # a dominant key just outside the window must NOT be seen
            k = torch.randn(S, nkv, hd) * 0.1
            direction = torch.ones(hd) / math.sqrt(hd)
            k[lo - 1] = 30.0 * direction
            q = (30.0 * direction).expand(1, nq, hd).clone()
            v = torch.randn(S, nkv, hd)
            k_pool, v_pool, tables = paged_cache([k], [v], P, dtype, DEV)
            got = ops.paged_attention_generic(q.reshape(1, -1).to(DEV, dtype), k_pool, v_pool,
                                              torch.tensor([S - 1], dtype=torch.int32, device=DEV),
                                              torch.zeros(1, dtype=torch.int32, device=DEV), table_tensor(tables, DEV),
                                              P, nq, nkv, hd, 1.0, window).float().cpu().view(nq, hd)
            assert (got[0] - v[lo - 1, 0]).abs().max() > 0.1


def test_sampler_kernel_against_the_plain_sampler(ops):
    from ullm_amd.sampling import Sampler, SamplingParams
    torch.manual_seed(7)
    sampler = Sampler(torch.device(DEV))
    configs = [(0.0, -1, 1.0, 0.0), (0.7, -1, 1.0, 0.0), (1.0, 5, 1.0, 0.0), (1.3, -1, 0.8, 0.0), (1.0, -1, 1.0, 0.1),
               (0.9, 20, 0.9, 0.05), (1.0, 1, 1.0, 0.0), (1.0, -1, 0.01, 0.0), (1.0, 2000, 1.0, 0.0)]
    for V in (503, 1537, 4100):            # 4100: rows aligned for the 16-byte path
        mismatches = 0
        for trial in range(5):
            logits = torch.randn(len(configs), V) * 3
            ps = [SamplingParams(temperature=c[0], top_k=c[1], top_p=c[2], min_p=c[3]) for c in configs]
            seeds = [trial * 100 + i for i in range(len(configs))]
            pos = [trial * 7 + i for i in range(len(configs))]
            got = sampler.sample(logits.to(DEV), ps, seeds, pos)
            want = [plain.sample_token(logits[i], *configs[i], seeds[i], pos[i]) for i in range(len(configs))]
            mismatches += sum(g != w for g, w in zip(got, want))
            # the same row in another batch position draws the same token
            again = sampler.sample(logits.flip(0).contiguous().to(DEV), ps[::-1], seeds[::-1], pos[::-1])
            assert again[::-1] == got
        assert mismatches == 0
    # ties: greedy takes the first index of the maximum
    logits = torch.zeros(2, 300)
    logits[0, [40, 7, 200]] = 5.0
    logits[1, 299] = 1.0
    assert sampler.sample(logits.to(DEV), [SamplingParams(temperature=0.0)] * 2, [0, 0], [0, 0]) == [7, 299]
    # frequencies follow the probabilities
    logits = torch.tensor([[0.0, 1.0, 2.0, -1.0, 0.5]])
    probs = torch.softmax(logits[0], -1)
    n = 4000
    rows = logits.expand(n, 5).contiguous().to(DEV)
    got = sampler.sample(rows, [SamplingParams(temperature=1.0)] * n, [99] * n, list(range(n)))
    counts = torch.bincount(torch.tensor(got), minlength=5).float()
    assert float(((counts - n * probs) ** 2 / (n * probs)).sum()) < 25.0


def test_sampler_with_a_small_top_k_over_a_large_vocabulary(ops):
    """Top-k with a small k, and top-p alone on a peaked row, gather the few values that can matter and
    filter those; rows where that cannot work (a large k, a flat row under top-p alone) find their thresholds by
    bins of the distance from the maximum, and where that cannot work either (many equal values around the k-th
    largest, the k-th largest far below the maximum) by halving over the whole vocabulary.  Either way the token
    is one the plain sampler may draw."""
    from ullm_amd.sampling import Sampler, SamplingParams
    torch.manual_seed(17)
    sampler = Sampler(torch.device(DEV))
    configs = [(0.6, 20, 0.95, 0.0), (1.0, 5, 1.0, 0.0), (0.8, 50, 0.9, 0.02), (1.0, 1000, 1.0, 0.0), (1.2, 1, 1.0, 0.0),
               (0.7, 20, 0.5, 0.0), (1.0, 1024, 0.99, 0.0), (1.0, 1025, 1.0, 0.0),
               (0.7, -1, 0.9, 0.0), (1.0, 0, 0.5, 0.02), (0.5, -1, 0.99, 0.0),        # top-p alone
               (1.0, 5000, 1.0, 0.0), (0.9, 3000, 0.8, 0.05), (1.3, 20000, 0.95, 0.0)]  # thresholds far down the row: by bins
    whole_rows = Sampler(torch.device(DEV), cut_rows=False)    # one block per row, no parts
    for V in (32000, 151936, 50257):       # 50257: rows not aligned for 16-byte loads
        masked = torch.randn(len(configs), V) * 3
        masked[:, 5000:27000] = float("-inf")                            # whole parts of a row without weight
        masked[:, -2000:] = float("-inf")
        kinds = {
            "masked": masked,
            "spread": torch.randn(len(configs), V) * 3,
            "peaked": torch.randn(len(configs), V) * 8,
            "flat": torch.randn(len(configs), V) * 0.01,                     # all within a hair of the maximum
            "ties": (torch.randn(len(configs), V) * 2).round(),              # many equal values: too many candidates
            "zeros of both signs": torch.where(torch.rand(len(configs), V) < 0.5, (torch.randn(len(configs), V) * 0.3).round(),
                                               torch.randn(len(configs), V) - 3.0),    # -0.0 and +0.0 are one value: the k-th largest is among them
            "far": torch.cat([torch.tensor([[50.0, 49.25, 48.5]]).expand(len(configs), 3),
                              torch.randn(len(configs), V - 3)], 1),           # the k-th largest far below the maximum
        }
        for name, logits in kinds.items():
            ps = [SamplingParams(temperature=c[0], top_k=c[1], top_p=c[2], min_p=c[3]) for c in configs]
            seeds = [7 + i for i in range(len(configs))]
            pos = [3 * i for i in range(len(configs))]
            got = sampler.sample(logits.to(DEV), ps, seeds, pos)
            for i, c in enumerate(configs):
                if name in ("ties", "zeros of both signs") and c[2] < 1.0:
                    continue       # which of several equal values top-p drops follows the reference's sort; here all or none
                assert got[i] in plain.sample_token_set(logits[i], *c, seeds[i], pos[i]), (V, name, c, got[i])
            again = sampler.sample(logits.flip(0).contiguous().to(DEV), ps[::-1], seeds[::-1], pos[::-1])
            assert again[::-1] == got
            whole = whole_rows.sample(logits.to(DEV), ps, seeds, pos)
            for i, c in enumerate(configs):
                if name in ("ties", "zeros of both signs") and c[2] < 1.0:
                    continue
                assert whole[i] in plain.sample_token_set(logits[i], *c, seeds[i], pos[i]), (V, name, c, whole[i])


def test_sampler_rows_cut_into_parts(ops):
    """Every setting but greedy and a top-k above 64 takes sums and candidates from parts of the row that a first
    kernel makes (top-p and min-p without top-k where what they keep lies within the 64 largest values of every part); the token is one the plain sampler may draw, whatever the row looks like and wherever in it the
    weight lies, and the same as in another batch position."""
    from ullm_amd.sampling import Sampler, SamplingParams
    torch.manual_seed(23)
    sampler = Sampler(torch.device(DEV))
    configs = [(0.7, -1, 1.0, 0.0), (1.0, 0, 1.0, 0.0), (1.5, -1, 1.0, 0.0), (0.6, 20, 0.95, 0.0), (1.0, 64, 1.0, 0.0),
               (0.8, 50, 0.9, 0.02), (1.0, 1, 1.0, 0.0), (0.3, 3, 1.0, 0.1), (1.0, 65, 1.0, 0.0),
               (0.7, -1, 0.9, 0.0), (0.25, 0, 0.5, 0.02), (1.0, -1, 0.999, 0.0),        # top-p without top-k
               (0.8, -1, 1.0, 0.05), (1.0, 0, 1.0, 0.9), (0.5, -1, 1.0, 1e-6),           # min-p alone
               (0.6, 0, 1.0, 1.0), (7.0, 20, 1.0, 1.0), (0.7, 2000, 1.0, 1.0)]           # a min-p of one: the ties for the maximum
    for V in (10240, 10244, 40960, 151936, 327680, 327684):      # one part exactly, one value into the next, the most parts, too many
        rows = {
            "spread": torch.randn(len(configs), V) * 3,
            "weight at the end": torch.cat([torch.randn(len(configs), V - 8) - 30.0, torch.randn(len(configs), 8) * 2], 1),
            "weight at a part's edge": torch.full((len(configs), V), -40.0),
            "equal values": torch.full((len(configs), V), 7.3),             # 7.3 / temperature is no exact product
            "several largest": torch.randn(len(configs), V) * 2,
            "the largest all in one part": torch.randn(len(configs), V),
            "peaked": torch.randn(len(configs), V) * 12,                     # a nucleus of few values
        }
        edge = min(10236, V - 8)
        rows["weight at a part's edge"][:, edge:edge + 8] = torch.randn(len(configs), 8)
        rows["the largest all in one part"][:, 3000:3100] += 20.0
        rows["several largest"][:, [5, 4097, V // 2, V - 1]] = 12.7
        for name, logits in rows.items():
            ps = [SamplingParams(temperature=c[0], top_k=c[1], top_p=c[2], min_p=c[3]) for c in configs]
            seeds = [11 + i for i in range(len(configs))]
            for trial in range(3):
                pos = [trial * 5 + i for i in range(len(configs))]
                got = sampler.sample(logits.to(DEV), ps, seeds, pos)
                for i, c in enumerate(configs):
                    if name in ("equal values", "several largest") and c[2] < 1.0:
                        continue   # which of several equal values top-p drops follows the reference's sort; here all or none
                    assert got[i] in plain.sample_token_set(logits[i], *c, seeds[i], pos[i]), (V, name, c, got[i])
                again = sampler.sample(logits.flip(0).contiguous().to(DEV), ps[::-1], seeds[::-1], pos[::-1])
                assert again[::-1] == got


MFMA_CASES = [dict(nq=8, nkv=2, hd=32, P=16, lens=[(1, 1), (1, 37), (1, 300), (1, 64)], window=0),
              dict(nq=32, nkv=8, hd=128, P=16, lens=[(1, 1153), (1, 31), (1, 32), (1, 33)], window=0),
              dict(nq=8, nkv=1, hd=64, P=32, lens=[(1, 500), (1, 97)], window=0),
              dict(nq=40, nkv=2, hd=64, P=16, lens=[(1, 130), (1, 17)], window=0),          # 20 heads per kv head
              dict(nq=4, nkv=4, hd=96, P=64, lens=[(1, 200), (1, 64)], window=0),
              dict(nq=6, nkv=2, hd=256, P=16, lens=[(1, 77)], window=0),
              dict(nq=8, nkv=2, hd=64, P=16, lens=[(1, 300), (1, 40), (1, 9)], window=50),
              dict(nq=8, nkv=2, hd=32, P=16, lens=[(5, 5), (33, 70), (16, 16), (2, 130), (17, 49)], window=0),
              dict(nq=32, nkv=8, hd=128, P=16, lens=[(100, 100), (7, 260)], window=0),
              dict(nq=32, nkv=16, hd=32, P=16, lens=[(70, 70), (33, 90), (1, 5)], window=0),      # kv heads 2 x 8
              dict(nq=6, nkv=2, hd=64, P=32, lens=[(40, 90), (3, 3)], window=21),
              dict(nq=10, nkv=2, hd=96, P=16, lens=[(45, 45), (2, 66)], window=0),       # 5 heads per kv head: 4 + 1 waves
              dict(nq=3, nkv=3, hd=256, P=16, lens=[(37, 80)], window=0),               # one head per kv head
              dict(nq=4, nkv=1, hd=128, P=16, lens=[(40, 1200), (64, 64)], window=0),   # page ids refetched past 1024 keys
              dict(nq=4, nkv=2, hd=64, P=48, lens=[(50, 1100)], window=300),
              dict(nq=2, nkv=2, hd=32, P=16, lens=[(2200, 2200), (70, 70)], window=0),  # 72 tiles: three rounds of blocks
              dict(nq=8, nkv=2, hd=32, P=16, lens=[(1, 45), (9, 40), (1, 200), (20, 20), (1, 1)], window=0),  # mixed
              dict(nq=8, nkv=2, hd=32, P=16, lens=[(1, 45), (9, 40), (1, 200), (20, 50)], window=13)]


@pytest.mark.parametrize("case", MFMA_CASES)
def test_attention_on_the_matrix_cores(ops, case):
    """Decoded tokens (split over the keys and reduced), prompt portions, and both in one batch."""
    torch.manual_seed(8)
    dtype = torch.bfloat16
    nq, nkv, hd, P, window = (case[k] for k in ("nq", "nkv", "hd", "P", "window"))
    assert ops.attention_mfma_supports(dtype, hd, P, nq, nkv)
    rnd = lambda *s: torch.randn(*s).to(dtype).float()   # noqa: E731
    ks = [rnd(S, nkv, hd) for _, S in case["lens"]]
    vs = [rnd(S, nkv, hd) for _, S in case["lens"]]
    qs = [rnd(n, nq, hd) for n, _ in case["lens"]]
    k_pool, v_pool, tables = paged_cache(ks, vs, P, dtype, DEV)          # unused rows are NaN
    positions = torch.cat([torch.arange(S - n, S) for n, S in case["lens"]]).int().to(DEV)
    entry = torch.cat([torch.full((n,), b) for b, (n, _) in enumerate(case["lens"])]).int().to(DEV)
    q = torch.cat(qs).reshape(-1, nq * hd).to(DEV, dtype)
    scale = hd ** -0.5
    want = reference_attention(qs, ks, vs, scale, window).reshape(-1, nq * hd)
    bt = table_tensor(tables, DEV)
    dec, tiles, t0, max_kv = [], [], 0, 0
    for n, S in case["lens"]:
        if n == 1:
            dec.append(t0)
            max_kv = max(max_kv, S)
        else:
            for f in range(0, n, ops.PREFILL_TILE):
                tiles += [t0 + f, min(ops.PREFILL_TILE, n - f)]
        t0 += n
    # prompt tiles: two halves of a block sharing the keys, one block taking all, and the chooser with
    # figures that send it either way
    # (11, 12: the kernel that stages tiles in registers, also where head size 128 has the one that loads them
    # straight to shared memory)
    halves = ((0, {}), (1, {}), (2, {}), (0, dict(keys_total=10 ** 9, keys_max=1)), (0, dict(keys_total=1, keys_max=10 ** 6)),
              (11, {}), (12, {}))
    for i, (splits, waves) in enumerate(((0, 0), (1, 4), (1, 8), (2, 8), (3, 4), (7, 8), (1, 1), (2, 1))):
        out = torch.full((q.shape[0], nq * hd), float("nan"), dtype=dtype, device=DEV)
        if dec:
            ops.attention_decode_mfma(q, out, k_pool, v_pool, torch.tensor(dec, dtype=torch.int32, device=DEV),
                                      len(dec), positions, entry, bt, P, nq, nkv, hd, scale, window, max_kv,
                                      splits=splits, waves=waves)
        if tiles:
            ops.attention_prefill_mfma(q, out, k_pool, v_pool, torch.tensor(tiles, dtype=torch.int32, device=DEV),
                                       len(tiles) // 2, positions, entry, bt, P, nq, nkv, hd, scale, window,
                                       halves=halves[i % len(halves)][0], **halves[i % len(halves)][1])
        assert not torch.isnan(out).any()
        assert (out.float().cpu() - want).abs().max() <= tol(dtype, want), (splits, waves, halves[i % len(halves)])
        if not dec and i + 1 >= len(halves):
            break


@pytest.mark.parametrize("row", [(5,), (7, 3), (64,), (1,), (4, 1000)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.uint8])
def test_state_rows_of_requests_that_start_afresh_are_zeroed(ops, row, dtype):
    """Rows of any size and type (16-, 4- and 1-byte words): only the slots of entries that start at 0 are
    zeroed, slots outside the tensor are ignored, nothing else is touched."""
    torch.manual_seed(1)
    slots = 9
    state = (torch.rand((slots,) + row, device=DEV) * 200 + 1).to(dtype)
    before = state.clone()
    entry_slot = torch.tensor([3, 0, 8, 5, 11, 2], dtype=torch.int32, device=DEV)
    entry_start = torch.tensor([0, 7, 0, 1, 0, 0], dtype=torch.int32, device=DEV)
    ops.zero_fresh_rows(state, entry_slot, entry_start, 5)                  # the sixth entry is not part of the batch
    for s_ in range(slots):
        want = torch.zeros_like(before[s_]) if s_ in (3, 8) else before[s_]
        assert torch.equal(state[s_], want), s_
    # an odd base address: a view that starts one row further on
    if dtype == torch.uint8 and row == (5,):
        view = state[1:]
        ops.zero_fresh_rows(view, torch.tensor([0], dtype=torch.int32, device=DEV), torch.tensor([0], dtype=torch.int32, device=DEV), 1)
        assert int(state[1].sum()) == 0 and torch.equal(state[2], before[2])


@pytest.mark.parametrize("cols", [503, 1024, 151936])
def test_rows_gathered_by_an_index_on_the_device(ops, cols):
    torch.manual_seed(2)
    src = torch.randn(7, cols + 8, device=DEV)[:, :cols]                    # rows with a stride of their own
    index = torch.tensor([6, 0, 3, 3, 9, -1], dtype=torch.int32, device=DEV)
    got = ops.gather_rows(src, index)
    assert got.shape == (6, cols)
    assert torch.equal(got[:4], src[[6, 0, 3, 3]]) and float(got[4:].abs().max()) == 0.0


FUSED_CASES = [dict(nq=32, nkv=8, hd=128, P=16, lens=[1153, 31, 32, 33, 1], window=0, norm=True, rope=True),
               dict(nq=8, nkv=2, hd=64, P=16, lens=[300, 40, 9, 17, 48], window=50, norm=True, rope=True),
               dict(nq=40, nkv=2, hd=64, P=32, lens=[130, 97], window=0, norm=False, rope=True),      # 20 heads per kv head
               dict(nq=6, nkv=2, hd=256, P=16, lens=[77, 160], window=0, norm=True, rope=False),
               dict(nq=4, nkv=1, hd=128, P=48, lens=[1200, 64, 49], window=0, norm=False, rope=False),
               # three shapes that a random search once reported: four-wave merge at head size 256, twelve heads per
               # kv head in one group of 16 columns over a long context, three heads per kv head cut in three
               dict(nq=48, nkv=8, hd=256, P=16, lens=[861, 906], window=0, norm=True, rope=True),
               dict(nq=96, nkv=8, hd=64, P=48, lens=[2492], window=0, norm=True, rope=True),
               dict(nq=6, nkv=2, hd=128, P=48, lens=[1789], window=0, norm=True, rope=True),
               # a request whose keys end with a tile's last key: the kernel of its own takes that tile without tests
               # per score, the one that holds the newest key itself with them; both must round alike
               dict(nq=24, nkv=2, hd=128, P=16, lens=[1643, 353, 1384, 25, 32], window=0, norm=True, rope=False)]


@pytest.mark.parametrize("case", FUSED_CASES)
def test_decode_attention_with_norm_rotation_and_cache_write_folded_in(ops, case):
    """A step of single new tokens through one kernel: against the plain formulas, and against the two
    kernels it stands for (the cache it leaves must be the one they leave).  The last entry of the batch is
    padding as a captured graph has it: position 0, no page; nothing may be written for it."""
    torch.manual_seed(12)
    dtype = torch.bfloat16
    nq, nkv, hd, P, window = (case[k] for k in ("nq", "nkv", "hd", "P", "window"))
    eps, theta, scale = 1e-5, 5000.0, hd ** -0.5
    rot, style = (hd, 1) if case["rope"] else (0, 0)
    assert ops.attention_decode_fused_supports(dtype, hd, P, nq, nkv, rot, style)
    assert not ops.attention_decode_fused_supports(dtype, hd, P, nq, nkv, hd // 2, 1)      # part of the head rotated
    assert not ops.attention_decode_fused_supports(dtype, hd, P, nq, nkv, hd, 2)           # adjacent pairs
    assert not ops.attention_decode_fused_supports(dtype, 96, P, 4, 4, 96, 1)
    rnd = lambda *s: torch.randn(*s).to(dtype).float()   # noqa: E731
    lens = case["lens"]
    B = len(lens) + 1
    # the cache so far: S - 1 keys per request; the page of the new key exists, its row is unwritten (NaN)
    ks = [rnd(S, nkv, hd) for S in lens]
    vs = [rnd(S, nkv, hd) for S in lens]
    k_pool, v_pool, tables = paged_cache(ks, vs, P, dtype, DEV)
    for b, S in enumerate(lens):
        page, row = tables[b][(S - 1) // P], (S - 1) % P
        k_pool[page, :, row] = float("nan")
        v_pool[page, :, :, row] = float("nan")
    positions = torch.tensor([S - 1 for S in lens] + [0], dtype=torch.int32, device=DEV)
    entry = torch.arange(B, dtype=torch.int32, device=DEV)
    bt = table_tensor(tables + [[]], DEV)
    qkv = rnd(B, (nq + 2 * nkv) * hd)
    qg = (1 + 0.2 * torch.randn(hd)) if case["norm"] else None
    kg = (1 + 0.2 * torch.randn(hd)) if case["norm"] else None
    table = None
    if case["rope"]:
        inv = 1.0 / (theta ** (torch.arange(0, rot, 2, dtype=torch.float32) / rot))
        ang = torch.arange(max(lens) + 3, dtype=torch.float32)[:, None] * inv[None]
        table = torch.cat((ang.cos(), ang.sin()), -1).contiguous().to(DEV)
    dev = lambda t: None if t is None else t.to(DEV)     # noqa: E731
    order = sorted(range(B), key=lambda b: -int(positions[b]))      # longest first, as the engine lists them
    dec = torch.tensor(order, dtype=torch.int32, device=DEV)
    max_kv = max(lens)
    # the plain formulas
    x = qkv[:len(lens)]
    q = x[:, :nq * hd].view(-1, nq, hd)
    k = x[:, nq * hd:(nq + nkv) * hd].view(-1, nkv, hd)
    v = x[:, (nq + nkv) * hd:].view(-1, nkv, hd)
    if case["norm"]:
        q, k = plain.rms_norm(q, qg, eps), plain.rms_norm(k, kg, eps)
    if case["rope"]:
        cos, sin = plain.rope_cos_sin(positions[:len(lens)].cpu(), rot, theta)
        q, k = plain.apply_rope_concat_layout(q, cos, sin), plain.apply_rope_concat_layout(k, cos, sin)
    k, q = k.to(dtype).float(), q.to(dtype).float()
    full_k = [torch.cat((ks[b][:S - 1], k[b:b + 1])) for b, S in enumerate(lens)]
    full_v = [torch.cat((vs[b][:S - 1], v[b:b + 1])) for b, S in enumerate(lens)]
    want = reference_attention([q[b:b + 1] for b in range(len(lens))], full_k, full_v, scale, window).reshape(-1, nq * hd)
    # the two kernels
    k_two, v_two = k_pool.clone(), v_pool.clone()
    q_two = torch.empty(B, nq * hd, dtype=dtype, device=DEV)
    ops.qk_norm_rope_write(qkv.to(DEV, dtype), q_two, dev(qg), dev(kg), eps, table, rot, style, positions, entry, bt,
                           k_two, v_two, P, nq, nkv, hd, write_kv=True)
    out_two = torch.zeros(B, nq * hd, dtype=dtype, device=DEV)
    ops.attention_decode_mfma(q_two, out_two, k_two, v_two, dec, B, positions, entry, bt, P, nq, nkv, hd, scale, window, max_kv)
    two = out_two[:len(lens)].float().cpu()
    biggest = float(want.abs().max())
    for splits, waves in ((0, 0), (1, 1), (1, 4), (2, 8), (3, 4), (7, 1), (16, 1)):
        k_one, v_one = k_pool.clone(), v_pool.clone()
        out = torch.full((B, nq * hd), float("nan"), dtype=dtype, device=DEV)
        ops.attention_decode_fused(qkv.to(DEV, dtype), out, dev(qg), dev(kg), eps, table, rot, style, k_one, v_one, dec, B,
                                   positions, entry, bt, P, nq, nkv, hd, scale, window, max_kv, write_kv=True,
                                   splits=splits, waves=waves)
        got = out[:len(lens)].float().cpu()
        shape = f"splits {splits}, waves {waves}"
        assert not torch.isnan(got).any(), f"{shape}: NaN in the output"
        err = float((got - want).abs().max())
        assert err <= tol(dtype, want), f"{shape}: {err:.3e} from the plain formulas, bound {tol(dtype, want):.3e}"
        # the cache: the same rows written with the same bits (both kernels norm and rotate in one order)
        assert torch.equal(torch.isnan(k_one), torch.isnan(k_two)) and torch.equal(torch.isnan(v_one), torch.isnan(v_two)), \
            f"{shape}: other rows of the cache written than by the two kernels"
        assert torch.equal(torch.nan_to_num(v_one.float()), torch.nan_to_num(v_two.float())), f"{shape}: values differ"
        dk = (torch.nan_to_num(k_one.float()) - torch.nan_to_num(k_two.float())).abs()
        assert float(dk.max()) == 0.0, f"{shape}: keys differ from the two kernels' by up to {float(dk.max()):.3e}"
        # against the two kernels: the same queries and keys, so with the same cut of the keys the same bits;
        # with another cut the 32-bit sums differ by rounding and the result by one bfloat16 step at most
        d_two = float((got - two).abs().max())
        if (splits, waves) == (0, 0):
            assert d_two == 0.0, f"{shape}: {d_two:.3e} from the two kernels with the same cut of the keys"
        else:
            assert d_two <= 2.0 ** -7 * biggest, \
                f"{shape}: {d_two:.3e} from the two kernels, one bfloat16 step of the largest output is {2.0 ** -7 * biggest:.3e}"
        for b, S in enumerate(lens):
            page, row = tables[b][(S - 1) // P], (S - 1) % P
            kerr = float((k_one[page, :, row].float().cpu() - k[b]).abs().max())
            assert kerr <= tol(dtype, k), f"{shape}: stored key of request {b} is {kerr:.3e} from the plain formulas"
    # a layer that reads a cache another layer wrote: nothing is written, the cache's own newest key is used
    k_read, v_read = k_two.clone(), v_two.clone()
    out = torch.full((B, nq * hd), float("nan"), dtype=dtype, device=DEV)
    ops.attention_decode_fused(qkv.to(DEV, dtype), out, dev(qg), dev(kg), eps, table, rot, style, k_read, v_read, dec, B,
                               positions, entry, bt, P, nq, nkv, hd, scale, window, max_kv, write_kv=False)
    assert torch.equal(torch.nan_to_num(k_read.float()), torch.nan_to_num(k_two.float()))
    assert (out[:len(lens)].float().cpu() - want).abs().max() <= tol(dtype, want)


@pytest.mark.parametrize("hd", [64, 128])
def test_two_large_scores_half_a_unit_apart_weigh_the_same_in_prompt_and_decode_steps(ops, hd):
    """Two keys whose scores are near 50 in the units of the exponent and half a unit apart, with opposite
    values: the output is (2^0.5 - 1) / (2^0.5 + 1) of the values' size if the exponents are right to a few
    thousandths.  A scale that is rounded into the bfloat16 queries moves an exponent of 50 by up to 0.1 and the
    output by a fifth; scores scaled in 32-bit (as both kinds of kernel do) leave only the weights' own rounding
    to bfloat16.  Prompt tiles (every shape of launch) and the decode kernel must agree with the 64-bit result."""
    torch.manual_seed(4)
    dtype = torch.bfloat16
    nq, nkv, P, S, n = 2, 1, 16, 200, 40
    scale = hd ** -0.5
    unit = scale * 1.4426950408889634                     # an exponent's unit in terms of q . k
    u = torch.randn(hd)
    u /= u.norm()
    k = (torch.randn(S, nkv, hd) * 0.05)
    q = (torch.randn(n, nq, hd) * 0.05)
    size = (50.0 / unit) ** 0.5
    a_at, b_at = 37, 150
    k[a_at, 0] = size * u
    k[b_at, 0] = size * u * (49.5 / 50.0)
    q[-1, :] = size * u
    k, q = k.to(dtype).double(), q.to(dtype).double()
    v = torch.zeros(S, nkv, hd)
    v[a_at], v[b_at] = 1.0, -1.0
    scores = (k[:, 0] @ q[-1, 0]) * scale
    want = (torch.softmax(scores, 0)[:, None] * v[:, 0].double()).sum(0)
    assert 0.1 < float(want[0]) < 0.25 and 45 < float(scores.max()) * 1.4427 < 55      # the case is the one described
    k_pool, v_pool, tables = paged_cache([k.float()], [v], P, dtype, DEV)
    bt = table_tensor(tables, DEV)
    positions = torch.arange(S - n, S, dtype=torch.int32, device=DEV)
    entry = torch.zeros(n, dtype=torch.int32, device=DEV)
    qd = q.float().reshape(n, nq * hd).to(DEV, dtype)
    tiles = torch.tensor([x for f in range(0, n, ops.PREFILL_TILE) for x in (f, min(ops.PREFILL_TILE, n - f))],
                         dtype=torch.int32, device=DEV)
    for halves in ((1, 2, 11, 12) if hd == 128 else (1, 2)):
        out = torch.zeros(n, nq * hd, dtype=dtype, device=DEV)
        ops.attention_prefill_mfma(qd, out, k_pool, v_pool, tiles, tiles.numel() // 2, positions, entry, bt, P, nq, nkv, hd,
                                   scale, 0, halves=halves)
        err = float((out[-1, :hd].double().cpu() - want).abs().max())
        assert err <= 6e-3, f"prompt tiles, halves {halves}: {err:.4f} from {float(want[0]):.4f}"
    for splits, waves in ((1, 1), (2, 4), (3, 1)):
        out = torch.zeros(1, nq * hd, dtype=dtype, device=DEV)
        ops.attention_decode_mfma(qd[-1:].contiguous(), out, k_pool, v_pool, None, 1, positions[-1:].contiguous(),
                                  entry[:1], bt, P, nq, nkv, hd, scale, 0, S, splits=splits, waves=waves)
        err = float((out[0, :hd].double().cpu() - want).abs().max())
        assert err <= 6e-3, f"decode, {splits} x {waves}: {err:.4f} from {float(want[0]):.4f}"


def test_matrix_core_attention_finds_one_far_key_at_every_edge(ops):
    torch.manual_seed(9)
    dtype = torch.bfloat16
    nq, nkv, hd, P, S = 8, 2, 64, 16, 403
    for window in (0, 70):
        lo = 0 if window == 0 else S - window
        targets = sorted(t for t in {lo, lo + 1, (lo // P + 1) * P - 1, (lo // P + 1) * P, 31, 32, 255, 256, 383, 384,
                                     S - 2, S - 1} if t >= lo)
        for target in targets:
            for n in (1, 5):
                k = torch.randn(S, nkv, hd) * 0.1
                v = torch.randn(S, nkv, hd).to(dtype).float()
                q = torch.randn(n, nq, hd) * 0.1
                direction = torch.randn(hd)
                direction /= direction.norm()
                k[target] = 30.0 * direction
                q[-1] = 30.0 * direction
                k, q = k.to(dtype).float(), q.to(dtype).float()
                k_pool, v_pool, tables = paged_cache([k], [v], P, dtype, DEV, seed=target)
                positions = torch.arange(S - n, S).int().to(DEV)
                entry = torch.zeros(n, dtype=torch.int32, device=DEV)
                qd = q.reshape(n, -1).to(DEV, dtype)
                out = torch.zeros(n, nq * hd, dtype=dtype, device=DEV)
                bt = table_tensor(tables, DEV)
                if n == 1:
                    ops.attention_decode_mfma(qd, out, k_pool, v_pool, None, 1, positions, entry, bt, P, nq, nkv, hd,
                                              1.0, window, S, splits=1 + target % 3, waves=8 if target % 2 else 4)
                else:
                    ops.attention_prefill_mfma(qd, out, k_pool, v_pool, torch.tensor([0, n], dtype=torch.int32, device=DEV),
                                               1, positions, entry, bt, P, nq, nkv, hd, 1.0, window)
                got = out.float().cpu().view(n, nq, hd)[-1]
                for h in range(nq):
                    assert (got[h] - v[target, h // 4]).abs().max() < 3e-2, (window, target, n, h)


def _dominant_key_problem(hd, S, n, target, nq=8, nkv=2, P=16, seed=0):
    """A cache of S keys in which key ``target`` is the only one the last of n queries looks at."""
    g = torch.Generator().manual_seed(1000 * seed + target)
    dtype = torch.bfloat16
    k = torch.randn(S, nkv, hd, generator=g) * 0.1
    v = torch.randn(S, nkv, hd, generator=g).to(dtype).float()
    q = torch.randn(n, nq, hd, generator=g) * 0.1
    direction = torch.randn(hd, generator=g)
    direction /= direction.norm()
    k[target] = 30.0 * direction
    q[-1] = 30.0 * direction
    k, q = k.to(dtype).float(), q.to(dtype).float()
    k_pool, v_pool, tables = paged_cache([k], [v], P, dtype, DEV, seed=target)
    positions = torch.arange(S - n, S).int().to(DEV)
    entry = torch.zeros(n, dtype=torch.int32, device=DEV)
    return q.reshape(n, -1).to(DEV, dtype), k_pool, v_pool, positions, entry, table_tensor(tables, DEV), v


@pytest.mark.parametrize("hd", [64, 128])
def test_matrix_core_attention_finds_one_far_key_beyond_a_thousand_keys(ops, hd):
    """The kernels fetch page ids 1024 keys at a time, cut a token's keys over waves and blocks, and (prompt
    tiles) over two halves of a block: one dominant key at every such seam must be found, by every shape of
    launch, and a dominant key one place before the window must not be seen.  Random data cannot show a
    dropped or doubled 16-key sub-block among two thousand keys; this can."""
    nq, nkv, P, S = 8, 2, 16, 2203
    decode_shapes = ((1, 1), (1, 4), (1, 8), (2, 8), (7, 8), (3, 1), (5, 4))          # (splits, waves)
    for window in (0, S - 1024, S - 1008, S - 2047, 300):
        lo = 0 if window == 0 else S - window
        seams = {lo, lo + 1, 1007, 1008, 1022, 1023, 1024, 1025, 1039, 1040, 2047, 2048, 2049, S - 33, S - 32, S - 2, S - 1}
        for target in sorted(t for t in seams if lo <= t < S):
            qd, k_pool, v_pool, positions, entry, bt, v = _dominant_key_problem(hd, S, 1, target, nq, nkv, P)
            for splits, waves in decode_shapes:
                out = torch.zeros(1, nq * hd, dtype=torch.bfloat16, device=DEV)
                ops.attention_decode_mfma(qd, out, k_pool, v_pool, None, 1, positions, entry, bt, P, nq, nkv, hd,
                                          1.0, window, S, splits=splits, waves=waves)
                got = out.float().cpu().view(nq, hd)
                for h in range(nq):
                    assert (got[h] - v[target, h // 4]).abs().max() < 3e-2, ("decode", window, target, splits, waves, h)
            for n in (5, 40):                     # one tile, and two tiles (the last query in the second)
                qd, k_pool, v_pool, positions, entry, bt, v = _dominant_key_problem(hd, S, n, target, nq, nkv, P, seed=1)
                tiles = [x for f in range(0, n, ops.PREFILL_TILE) for x in (f, min(ops.PREFILL_TILE, n - f))]
                for halves in (1, 2, 11, 12):
                    out = torch.zeros(n, nq * hd, dtype=torch.bfloat16, device=DEV)
                    ops.attention_prefill_mfma(qd, out, k_pool, v_pool, torch.tensor(tiles, dtype=torch.int32, device=DEV),
                                               len(tiles) // 2, positions, entry, bt, P, nq, nkv, hd, 1.0, window,
                                               halves=halves)
                    got = out.float().cpu().view(n, nq, hd)[-1]
                    for h in range(nq):
                        assert (got[h] - v[target, h // 4]).abs().max() < 3e-2, ("prompt", window, target, n, halves, h)
        if window:
            # the key one place before the window dominates every key inside it, and must not be seen
            target = lo - 1
            qd, k_pool, v_pool, positions, entry, bt, v = _dominant_key_problem(hd, S, 1, target, nq, nkv, P, seed=2)
            for splits, waves in decode_shapes:
                out = torch.zeros(1, nq * hd, dtype=torch.bfloat16, device=DEV)
                ops.attention_decode_mfma(qd, out, k_pool, v_pool, None, 1, positions, entry, bt, P, nq, nkv, hd,
                                          1.0, window, S, splits=splits, waves=waves)
                got = out.float().cpu().view(nq, hd)
                assert (got[0] - v[target, 0]).abs().max() > 0.1, ("decode sees past its window", window, splits, waves)
            qd, k_pool, v_pool, positions, entry, bt, v = _dominant_key_problem(hd, S, 5, target, nq, nkv, P, seed=3)
            for halves in (1, 2, 11, 12):
                out = torch.zeros(5, nq * hd, dtype=torch.bfloat16, device=DEV)
                ops.attention_prefill_mfma(qd, out, k_pool, v_pool, torch.tensor([0, 5], dtype=torch.int32, device=DEV), 1,
                                           positions, entry, bt, P, nq, nkv, hd, 1.0, window, halves=halves)
                got = out.float().cpu().view(5, nq, hd)[-1]
                assert (got[0] - v[target, 0]).abs().max() > 0.1, ("a prompt tile sees past its window", window, halves)


def test_prompt_attention_over_more_keys_than_its_page_table_holds(ops):
    """The prompt kernel for head size 128 keeps the page ids of 128 tiles (4096 keys) in shared memory and
    refills them on the way: a dominant key on either side of every refill (one block taking all keys: 4096,
    8192; two halves of a block: each half's own 4096th key) must be found, with and without a window, and all
    query rows must agree with a plain softmax over the keys."""
    hd, nq, nkv, P, S, n = 128, 4, 1, 16, 9001, 37
    for window in (0, 6000):
        lo = 0 if window == 0 else S - window
        half = lo // 32 * 32 + ((S - lo // 32 * 32 + 31) // 32 + 1) // 2 * 32       # first key of the second half
        seams = {lo, 4095, 4096, 4097, 8191, 8192, 8193, half - 1, half, half + 4095, half + 4096, S - 40, S - 1}
        for target in sorted(t for t in seams if lo <= t < S):
            qd, k_pool, v_pool, positions, entry, bt, v = _dominant_key_problem(hd, S, n, target, nq, nkv, P, seed=4)
            tiles = [x for f in range(0, n, ops.PREFILL_TILE) for x in (f, min(ops.PREFILL_TILE, n - f))]
            for halves in (1, 2, 12):
                out = torch.zeros(n, nq * hd, dtype=torch.bfloat16, device=DEV)
                ops.attention_prefill_mfma(qd, out, k_pool, v_pool, torch.tensor(tiles, dtype=torch.int32, device=DEV),
                                           len(tiles) // 2, positions, entry, bt, P, nq, nkv, hd, 1.0, window, halves=halves)
                got = out.float().cpu().view(n, nq, hd)
                if target <= S - n:            # visible to every query of the portion; the last query looks straight at it
                    for h in range(nq):
                        assert (got[-1, h] - v[target, 0]).abs().max() < 3e-2, (window, target, halves, h)
    # the same seams for a single decoded token, whose kernel fetches page ids 1024 keys at a time
    for target in (1023, 1024, 4095, 4096, 8191, 8192, S - 1):
        qd, k_pool, v_pool, positions, entry, bt, v = _dominant_key_problem(hd, S, 1, target, nq, nkv, P, seed=5)
        for splits, waves in ((1, 1), (1, 8), (2, 8), (16, 1), (5, 4)):
            out = torch.zeros(1, nq * hd, dtype=torch.bfloat16, device=DEV)
            ops.attention_decode_mfma(qd, out, k_pool, v_pool, None, 1, positions, entry, bt, P, nq, nkv, hd, 1.0, 0, S,
                                      splits=splits, waves=waves)
            got = out.float().cpu().view(nq, hd)
            for h in range(nq):
                assert (got[h] - v[target, 0]).abs().max() < 3e-2, ("decode", target, splits, waves, h)
    # random data, every query row against a plain softmax
    torch.manual_seed(6)
    k = torch.randn(S, nkv, hd).bfloat16().float()
    vv = torch.randn(S, nkv, hd).bfloat16().float()
    q = torch.randn(n, nq, hd).bfloat16().float()
    k_pool, v_pool, tables = paged_cache([k], [vv], P, torch.bfloat16, DEV, seed=3)
    positions = torch.arange(S - n, S).int().to(DEV)
    entry = torch.zeros(n, dtype=torch.int32, device=DEV)
    bt = table_tensor(tables, DEV)
    tiles = torch.tensor([x for f in range(0, n, ops.PREFILL_TILE) for x in (f, min(ops.PREFILL_TILE, n - f))], dtype=torch.int32, device=DEV)
    scale = hd ** -0.5
    for window in (0, 6000):
        scores = torch.einsum("qhd,kd->qhk", q, k[:, 0]) * scale
        pos = torch.arange(S - n, S)[:, None, None]
        keys = torch.arange(S)[None, None, :]
        hidden = (keys > pos) | ((keys <= pos - window) if window else torch.zeros_like(keys > pos))
        want = torch.einsum("qhk,kd->qhd", torch.softmax(scores.masked_fill(hidden, float("-inf")), -1), vv[:, 0]).reshape(n, -1)
        for halves in (0, 1, 2):
            out = torch.zeros(n, nq * hd, dtype=torch.bfloat16, device=DEV)
            ops.attention_prefill_mfma(q.reshape(n, -1).to(DEV, torch.bfloat16), out, k_pool, v_pool, tiles, tiles.numel() // 2,
                                       positions, entry, bt, P, nq, nkv, hd, scale, window, halves=halves)
            assert (out.float().cpu() - want).abs().max() <= tol(torch.bfloat16, want), (window, halves)


@pytest.mark.parametrize("dtype,hd,nq", [(torch.bfloat16, 128, 8), (torch.float32, 64, 4)])
def test_cache_pools_beyond_four_gibi_elements(ops, dtype, hd, nq):
    """A cache sized for this GPU's memory: pools of five gibi-elements each (10 and 20 GiB) with the live pages
    at their far end, where 32-bit element and byte offsets have wrapped.  Every kernel that touches the cache
    (rotary + write, decode and prompt attention on the matrix cores, the fused decode step, the general
    attention) must give, bit for bit, what it gives on a small pool, and write nowhere else."""
    free, _ = torch.cuda.mem_get_info()
    if free < (48 << 30):
        pytest.skip("needs 48 GiB of free device memory")
    torch.manual_seed(3)
    nkv, P, lens = 2, 16, [(1, 300), (1, 37), (40, 200), (70, 70)]
    rnd = lambda *s: torch.randn(*s).to(dtype).float()   # noqa: E731
    ks, vs = [rnd(S, nkv, hd) for _, S in lens], [rnd(S, nkv, hd) for _, S in lens]
    k_small, v_small, tables = paged_cache(ks, vs, P, dtype, DEV, fill=0.0)
    n_small, big_pages = k_small.shape[0], (5 << 30) // (nkv * P * hd)
    shift = big_pages - n_small
    k_big = torch.zeros((big_pages, nkv, P, hd), dtype=dtype, device=DEV)
    v_big = torch.zeros((big_pages, nkv, hd, P), dtype=dtype, device=DEV)
    k_big[shift:], v_big[shift:] = k_small, v_small
    positions = torch.cat([torch.arange(S - n, S) for n, S in lens]).int().to(DEV)
    entry = torch.cat([torch.full((n,), b) for b, (n, _) in enumerate(lens)]).int().to(DEV)
    T = positions.numel()
    qkv = rnd(T, (nq + 2 * nkv) * hd).to(DEV, dtype)
    gain = (1 + 0.1 * torch.randn(hd)).to(DEV)
    inv = 1.0 / (10000.0 ** (torch.arange(0, hd, 2, dtype=torch.float32) / hd))
    ang = torch.arange(302, dtype=torch.float32)[:, None] * inv[None]
    table = torch.cat((ang.cos(), ang.sin()), -1).contiguous().to(DEV)
    dec = torch.tensor([0, 1], dtype=torch.int32, device=DEV)
    tiles = torch.tensor([x for t0, n in ((2, 40), (42, 70)) for f in range(0, n, ops.PREFILL_TILE)
                          for x in (t0 + f, min(ops.PREFILL_TILE, n - f))], dtype=torch.int32, device=DEV)
    scale, results = hd ** -0.5, []
    for kp, vp, tb in ((k_small.clone(), v_small.clone(), tables), (k_big, v_big, [[p + shift for p in t] for t in tables])):
        bt, res = table_tensor(tb, DEV), {}
        q = torch.empty(T, nq * hd, dtype=dtype, device=DEV)
        ops.qk_norm_rope_write(qkv, q, gain, gain, 1e-6, table, hd, 1, positions, entry, bt, kp, vp, P, nq, nkv, hd, write_kv=True)
        res["q"] = q
        new = lambda: torch.zeros(T, nq * hd, dtype=dtype, device=DEV)   # noqa: E731
        if dtype == torch.bfloat16:
            for splits, waves in ((0, 0), (1, 4), (3, 1)):
                res[f"decode {splits}x{waves}"] = out = new()
                ops.attention_decode_mfma(q, out, kp, vp, dec, 2, positions, entry, bt, P, nq, nkv, hd, scale, 0, 300,
                                          splits=splits, waves=waves)
            for halves in (1, 2, 11, 12):
                res[f"prompt {halves}"] = out = new()
                ops.attention_prefill_mfma(q, out, kp, vp, tiles, tiles.numel() // 2, positions, entry, bt, P, nq, nkv, hd,
                                           scale, 0, halves=halves)
            res["fused"] = out = new()
            ops.attention_decode_fused(qkv, out, gain, gain, 1e-6, table, hd, 1, kp, vp, dec, 2, positions, entry, bt, P, nq,
                                       nkv, hd, scale, 0, 300, write_kv=True)
        res["general"] = ops.paged_attention_generic(q, kp, vp, positions, entry, bt, P, nq, nkv, hd, scale, 0, out=new())
        res["keys"], res["values"] = kp[-n_small:].clone(), vp[-n_small:].clone()
        results.append(res)
    for name, small in results[0].items():
        assert float(small.float().abs().max()) > 0 and torch.equal(small, results[1][name]), name
    assert float(k_big[:shift].abs().max()) == 0 and float(v_big[:shift].abs().max()) == 0
    del k_big, v_big, kp, vp, results
    torch.cuda.empty_cache()           # the pools go back to the device, not to torch's cache


def test_matrix_core_attention_with_scores_that_climb(ops):
    """The reference value of the exponentials follows the running maximum only in steps: scores that
    rise a little with every tile (so it lags, then jumps) and scores that fall must both come out right."""
    torch.manual_seed(12)
    dtype = torch.bfloat16
    nq, nkv, hd, P, S = 4, 2, 32, 16, 640
    for slope in (0.09, -0.09, 0.4):                      # natural-log units per key: 2.9, -2.9, 12.8 per 32-key tile
        k = torch.randn(S, nkv, hd) * 0.05
        k[:, :, 0] = slope * torch.arange(S).float()[:, None]
        v = torch.randn(S, nkv, hd)
        k, v = k.to(dtype).float(), v.to(dtype).float()
        for n in (1, 40):
            q = torch.randn(n, nq, hd) * 0.05
            q[:, :, 0] = 1.0
            q = q.to(dtype).float()
            want = reference_attention([q], [k], [v], 1.0, 0).reshape(n, nq * hd)
            k_pool, v_pool, tables = paged_cache([k], [v], P, dtype, DEV)
            positions = torch.arange(S - n, S).int().to(DEV)
            entry = torch.zeros(n, dtype=torch.int32, device=DEV)
            qd = q.reshape(n, -1).to(DEV, dtype)
            out = torch.zeros(n, nq * hd, dtype=dtype, device=DEV)
            bt = table_tensor(tables, DEV)
            if n == 1:
                ops.attention_decode_mfma(qd, out, k_pool, v_pool, None, 1, positions, entry, bt, P, nq, nkv, hd,
                                          1.0, 0, S, splits=1, waves=4)
            else:
                tiles = [x for f in range(0, n, ops.PREFILL_TILE) for x in (f, min(ops.PREFILL_TILE, n - f))]
                ops.attention_prefill_mfma(qd, out, k_pool, v_pool, torch.tensor(tiles, dtype=torch.int32, device=DEV),
                                           len(tiles) // 2, positions, entry, bt, P, nq, nkv, hd, 1.0, 0)
            assert (out.float().cpu() - want).abs().max() <= tol(dtype, want), (slope, n)


@pytest.mark.parametrize("shape", [(1, 48, 64), (8, 503, 96), (16, 256, 4096), (17, 100, 224), (33, 64, 1032),
                                   (64, 130, 520), (5, 4096, 128), (3, 16, 8), (2, 9496, 72)])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
def test_gemm_skinny(ops, shape, out_dtype):
    torch.manual_seed(10)
    M, N, K = shape
    a = torch.randn(M, K, device=DEV).bfloat16()
    w = torch.randn(N, K, device=DEV).bfloat16()
    b = torch.randn(N, device=DEV)
    want = (a.double() @ w.double().T + b.double()).float()
    got = ops.gemm_skinny(a, w, b, out_dtype=out_dtype)
    assert got.dtype == out_dtype
    for nt, waves in ((1, 1), (2, 2), (2, 16), (4 if M > 16 else 2, 4)):
        other = ops.gemm_skinny(a, w, b, out_dtype=out_dtype, nt=nt, waves=waves)
        assert (other.float() - got.float()).abs().max() <= 1e-2 * float(want.abs().max()), (nt, waves)
        if out_dtype == torch.float32:
            assert (other - want).abs().max() <= 2e-5 * float(want.abs().max()), (nt, waves)
    bound = (1e-2 if out_dtype == torch.bfloat16 else 2e-5) * float(want.abs().max())
    assert (got.float() - want).abs().max() <= bound
    assert torch.equal(ops.gemm_skinny(a, w, b, out_dtype=out_dtype), got)          # repeatable bit for bit
    # strided activations (a column slice of a wider buffer)
    wide = torch.randn(M, K + 64, device=DEV).bfloat16()
    wide[:, 32:32 + K] = a
    got2 = ops.gemm_skinny(wide[:, 32:32 + K], w, b, out_dtype=out_dtype)
    assert torch.equal(got2, got)


@pytest.mark.parametrize("shape", [(8, 200, 256), (3, 6144, 512), (16, 1000, 264), (20, 520, 128)])
def test_gemm_skinny_with_fewer_columns_a_block(ops, shape):
    """A block may own fewer columns of the result than its tiles hold (so that the blocks spread
    evenly over the compute units): every such split gives the same product, the folded forms too."""
    torch.manual_seed(16)
    M, N, K = shape
    a = torch.randn(M, K, device=DEV).bfloat16()
    w = (torch.randn(N, K, device=DEV) * 0.3).bfloat16()
    b = torch.randn(N, device=DEV)
    want = ops.gemm_skinny(a, w, b, out_dtype=torch.float32)
    ref = a.double().cpu() @ w.double().cpu().T + b.double().cpu()
    assert (want.double().cpu() - ref).abs().max() <= 2e-5 * float(ref.abs().max())
    stream0 = torch.randn(M, N, device=DEV)
    gain = 1.0 + 0.5 * torch.randn(K, device=DEV)
    hstream = torch.randn(M, K, device=DEV)
    for nt, rows in ((1, 4), (1, 12), (2, 20), (2, 24), (2, 28), (1, 16), (2, 32)):
        got = ops.gemm_skinny(a, w, b, out_dtype=torch.float32, nt=nt, rows=rows)
        assert torch.equal(got, want) or (got - want).abs().max() <= 2e-6 * float(want.abs().max()), (nt, rows)
        s1, s2 = stream0.clone(), stream0.clone()
        ops.gemm_skinny_add(a, w, s1, nt=nt)
        ops.gemm_skinny_add(a, w, s2, nt=nt, rows=rows)
        assert (s1 - s2).abs().max() <= 2e-6 * float(s1.abs().max()), (nt, rows)
        if M <= 16:
            n1 = ops.gemm_skinny_normed(hstream, gain, 1e-5, w, b, out_dtype=torch.float32, nt=nt)
            n2 = ops.gemm_skinny_normed(hstream, gain, 1e-5, w, b, out_dtype=torch.float32, nt=nt, rows=rows)
            assert (n1 - n2).abs().max() <= 2e-6 * float(n1.abs().max()), (nt, rows)
    inter = N // 2
    wgu = torch.cat([w[:inter], w[N - inter:]]).contiguous()
    g1 = ops.gemm_skinny_silu(a, wgu)
    for rows in (4, 12, 16):
        assert torch.equal(ops.gemm_skinny_silu(a, wgu, rows=rows), g1), rows
    with pytest.raises(Exception):
        ops.gemm_skinny(a, w, b, nt=1, rows=20)            # more than a tile holds
    with pytest.raises(Exception):
        ops.gemm_skinny(a, w, b, nt=2, rows=10)            # no multiple of 4


@pytest.mark.parametrize("shape", [(1, 64, 128), (8, 6144, 4096), (5, 100, 1032), (16, 328, 72), (3, 70000, 264),
                                   (13, 24, 5128)])
def test_gemm_skinny_with_the_norm_folded_in(ops, shape):
    """rmsnorm(stream) W^T, and silu(gate) * up of it, straight from the 32-bit residual stream: against the plain
    norm followed by the plain product.  The rows' scales differ by orders of magnitude, so that a
    sum of squares that leaks from one row into another, or a missing scale, shows."""
    torch.manual_seed(14)
    M, N, K = shape
    stream = torch.randn(M, K, device=DEV) * torch.logspace(-2, 2, M, device=DEV)[:, None]
    gain = 1.0 + 0.5 * torch.randn(K, device=DEV)
    w = (torch.randn(N, K, device=DEV) * 0.3).bfloat16()
    b = torch.randn(N, device=DEV)
    eps = 1e-3
    normed = plain.rms_norm(stream.cpu(), gain.cpu(), eps)
    want = normed @ w.float().cpu().T + b.cpu()
    for out_dtype in (torch.bfloat16, torch.float32):
        got = ops.gemm_skinny_normed(stream, gain, eps, w, b, out_dtype=out_dtype)
        assert got.dtype == out_dtype and got.shape == (M, N)
        # the inputs of the matrix cores are rounded to bfloat16 (2^-9 each way) as after a norm kernel of its own
        assert (got.float().cpu() - want).abs().max() <= 1e-2 * float(want.abs().max())
        assert torch.equal(ops.gemm_skinny_normed(stream, gain, eps, w, b, out_dtype=out_dtype), got)
        for nt, waves in ((1, 1), (2, 2), (1, 8), (2, 4)):
            other = ops.gemm_skinny_normed(stream, gain, eps, w, b, out_dtype=out_dtype, nt=nt, waves=waves)
            assert (other.float().cpu() - want).abs().max() <= 1e-2 * float(want.abs().max()), (nt, waves)
    # against the two kernels it replaces: the same but for where the rounding to bfloat16 falls
    two = ops.gemm_skinny(ops.add_rmsnorm(None, stream.clone(), gain, eps, torch.bfloat16), w, b, out_dtype=torch.float32)
    one = ops.gemm_skinny_normed(stream, gain, eps, w, b, out_dtype=torch.float32)
    assert (one - two).abs().max() <= 4e-3 * float(want.abs().max())
    # fewer rows of the same stream: every row as before, bit for bit
    if M > 1:
        fewer = ops.gemm_skinny_normed(stream[:M // 2], gain, eps, w, b, out_dtype=torch.float32)
        assert torch.equal(fewer, one[:M // 2])
    # a row of zeros: eps alone under the root, no NaN
    zeros = torch.zeros(2, K, device=DEV)
    assert torch.equal(ops.gemm_skinny_normed(zeros, gain, eps, w, out_dtype=torch.float32),
                       torch.zeros(2, N, device=DEV))
    inter = N // 2
    if inter:
        wgu = torch.cat([w[:inter], w[N - inter:]]).contiguous()
        want = plain.silu_and_mul(normed @ wgu.float().cpu().T)
        got = ops.gemm_skinny_normed(stream, gain, eps, wgu, silu=True)
        assert got.shape == (M, inter) and got.dtype == torch.bfloat16
        assert (got.float().cpu() - want).abs().max() <= 1e-2 * float(want.abs().max())


@pytest.mark.parametrize("shape", [(1, 64, 128, 96), (8, 4096, 1024, 6144), (5, 1032, 264, 100), (16, 328, 72, 520),
                                   (3, 5120, 200, 70000), (13, 24, 512, 36), (9, 8200, 64, 256)])
def test_a_norm_handed_from_one_product_to_the_next(ops, shape):
    """A product that adds into the 32-bit stream also leaves, for the norm that comes next, the stream times that
    norm's gain in bfloat16 and every block's share of the rows' sums of squares; the next product multiplies the
    former and scales its rows by the latter.  Against the plain add, norm and product, with rows whose scales
    differ by orders of magnitude (a sum that leaks into another row, or a share of the squares that is lost or
    counted twice, shows), widths (M, hidden, inner of the first, outputs of the second) that are no multiples of
    a block's columns, and more blocks than the lanes of the second product fetch at once."""
    torch.manual_seed(15)
    M, H, K, N = shape
    a = torch.randn(M, K, device=DEV).bfloat16()
    w1 = (torch.randn(H, K, device=DEV) * 0.1).bfloat16()
    stream0 = torch.randn(M, H, device=DEV) * torch.logspace(-2, 2, M, device=DEV)[:, None]
    gain = 1.0 + 0.5 * torch.randn(H, device=DEV)
    w2 = (torch.randn(N, H, device=DEV) * 0.3).bfloat16()
    b = torch.randn(N, device=DEV)
    eps = 1e-3
    for kw in (dict(nt=1, waves=1), dict(nt=2, waves=4), dict(nt=1, rows=12), dict(nt=2, rows=20), {}):
        plain_stream, stream = stream0.clone(), stream0.clone()
        ops.gemm_skinny_add(a, w1, plain_stream, **kw)
        scaled, squares = ops.gemm_skinny_add(a, w1, stream, next_gain=gain, **kw)
        assert torch.equal(stream, plain_stream), kw                       # the add itself is untouched
        assert scaled.dtype == torch.bfloat16 and torch.equal(scaled, (stream * gain).bfloat16()), kw
        assert squares.shape[0] == M and squares.shape[1] % 4 == 0
        want_sq = stream.double().pow(2).sum(-1)
        assert ((squares.double().sum(-1) - want_sq).abs() <= 1e-6 * want_sq).all(), kw
    normed = plain.rms_norm(stream.cpu(), gain.cpu(), eps)
    want = normed @ w2.float().cpu().T + b.cpu()
    bound = 1e-2 * float(want.abs().max())
    results = {"few rows": ops.gemm_skinny(scaled, w2, b, out_dtype=torch.float32, squares=squares, eps=eps),
               "few rows, one wave": ops.gemm_skinny(scaled, w2, b, out_dtype=torch.float32, squares=squares, eps=eps,
                                                     nt=1, waves=1),
               "few rows, two tiles": ops.gemm_skinny(scaled, w2, b, out_dtype=torch.float32, squares=squares, eps=eps,
                                                      nt=2, waves=2)}
    if ops.gemm_rows_supports(scaled, w2):
        results["rows"] = ops.gemm_rows(scaled, w2, b, squares=squares, eps=eps)
    for name, got in results.items():
        assert (got.float().cpu() - want).abs().max() <= bound, name
    # the same arithmetic as the norm folded into the product (x * gain rounded, the product, the scale): the same bits
    if ops.gemm_skinny_normed_supports(stream, gain, w2):
        folded = ops.gemm_skinny_normed(stream, gain, eps, w2, b, out_dtype=torch.float32)
        assert (results["few rows"] - folded).abs().max() <= 2e-6 * float(want.abs().max())
    # fewer rows of the same stream: every row as before, bit for bit (up to 8 rows and beyond them the lanes share
    # out the sums of squares differently: across that line the scale may differ in its last bit)
    for m in {M // 2, M - 1} - {0}:
        fewer = ops.gemm_skinny(scaled[:m], w2, b, out_dtype=torch.float32, squares=squares[:m].contiguous(), eps=eps)
        if (m <= 8) == (M <= 8):
            assert torch.equal(fewer, results["few rows"][:m]), m
        assert (fewer - results["few rows"][:m]).abs().max() <= 1e-6 * float(want.abs().max())
    inter = N // 2
    if inter:
        wgu = torch.cat([w2[:inter], w2[N - inter:]]).contiguous()
        want = plain.silu_and_mul(normed @ wgu.float().cpu().T)
        outs = {"few rows": ops.gemm_skinny_silu(scaled, wgu, squares=squares, eps=eps)}
        if ops.gemm_rows_supports(scaled, wgu, silu=True):
            outs["rows"] = ops.gemm_rows(scaled, wgu, silu=True, squares=squares, eps=eps)
        for name, got in outs.items():
            assert got.shape == (M, inter) and got.dtype == torch.bfloat16
            assert (got.float().cpu() - want).abs().max() <= 1e-2 * float(want.abs().max()), name
    # what the kernels refuse: more than one tile of rows, squares of another batch
    with pytest.raises(Exception):
        ops.gemm_skinny(scaled, w2, squares=squares[:, :2].contiguous(), eps=eps)
    with pytest.raises(Exception):
        ops.gemm_skinny(torch.cat([scaled] * 3)[:17].contiguous(), w2, squares=torch.ones(17, 4, device=DEV), eps=eps)


@pytest.mark.parametrize("shape", [(2, 2, 1536), (1, 4, 1000), (3, 2, 24), (7, 6, 72), (16, 4, 200), (5, 2, 520)])
def test_folded_norm_on_few_outputs_errs_by_the_rounding_of_its_inputs(ops, shape):
    """silu(gate) * up of rmsnorm(stream) for two to six outputs a row, inner sizes that are no multiple of a
    stage of 64.  With so few outputs all of them may lie near zero, far below the row's own size |x| |w|, and
    an error that is small against the row looks large against the outputs' maximum (a random search reported
    6e-2 and 1.2e-1 of that maximum for the first two shapes).  So the error is measured against a product in
    64-bit and bounded by what rounding x * gain to bfloat16 can do to each sum: independent errors of at most
    2^-9 |x_i w_i|, bounded here by 4 * 2^-9 * sqrt(sum (x_i w_i)^2), seven standard deviations.  A piece of
    eight values lost or taken twice at the end of K would be an error of a few |x_i w_i|, ten times that."""
    M, inter, K = shape
    for seed in range(40):
        torch.manual_seed(seed)
        stream = torch.randn(M, K, device=DEV) * 2
        gain = 1 + 0.1 * torch.randn(K, device=DEV)
        w = (torch.randn(2 * inter, K, device=DEV) * 0.05).bfloat16()
        eps = 1e-6
        s64, g64, w64 = stream.double().cpu(), gain.double().cpu(), w.double().cpu()
        xn = s64 * torch.rsqrt(s64.pow(2).mean(-1, keepdim=True) + eps) * g64               # [M, K]
        sums = xn @ w64.T                                                                    # [M, 2 I]
        d_sum = 4 * 2.0 ** -9 * torch.sqrt((xn.pow(2)) @ (w64.pow(2)).T) + 1e-6              # per sum
        gate, up = sums[:, :inter], sums[:, inter:]
        want = torch.nn.functional.silu(gate) * up
        # silu' lies in [-0.1, 1.1]; the result is rounded to bfloat16 (2^-8 of itself)
        bound = 1.1 * up.abs() * d_sum[:, :inter] + torch.nn.functional.silu(gate).abs() * d_sum[:, inter:] \
            + d_sum[:, :inter] * d_sum[:, inter:] + 2.0 ** -8 * want.abs() + 1e-6
        got = ops.gemm_skinny_normed(stream, gain, eps, w, silu=True).double().cpu()
        over = ((got - want).abs() / bound).max()
        assert float(over) <= 1.0, f"seed {seed}: error {float(over):.2f} times the bound from the inputs' rounding"
        plain_sums = ops.gemm_skinny_normed(stream, gain, eps, w, out_dtype=torch.float32).double().cpu()
        over = ((plain_sums - sums).abs() / d_sum).max()
        assert float(over) <= 1.0, f"seed {seed}: the sums err by {float(over):.2f} times the bound"


@pytest.mark.parametrize("shape", [(17, 256, 512), (33, 100, 4104), (48, 4100, 72), (64, 640, 2048), (5, 128, 8),
                                   (64, 4096, 1032), (40, 24, 12288), (65, 260, 520), (100, 128, 1096), (129, 512, 264),
                                   (200, 96, 4096), (256, 1032, 776)])
def test_gemm_partial_sums(ops, shape):
    """The product for 17 to 256 rows as a stack of partial sums over slices of K, and the add + norm
    kernel that adds the stack."""
    torch.manual_seed(12)
    M, N, K = shape
    a = torch.randn(M, K, device=DEV).bfloat16()
    w = (torch.randn(N, K, device=DEV) * 0.2).bfloat16()
    want = a.double().cpu() @ w.double().cpu().T
    stack = ops.gemm_partial_sums(a, w)
    assert stack.dtype == torch.float32 and stack.shape[1:] == (M, N) and stack.shape[0] >= 1
    assert (stack.sum(0).double().cpu() - want).abs().max() <= 2e-5 * float(want.abs().max()) + 1e-6
    assert torch.equal(ops.gemm_partial_sums(a, w), stack)                     # repeatable bit for bit
    fewer = ops.gemm_partial_sums(a[:M // 2 + 1], w)                             # the slices follow the matrix, not the batch
    assert fewer.shape[0] == stack.shape[0] and torch.equal(fewer, stack[:, :M // 2 + 1])
    # strided activations (a column slice of a wider buffer)
    wide = torch.randn(M, K + 64, device=DEV).bfloat16()
    wide[:, 32:32 + K] = a
    assert torch.equal(ops.gemm_partial_sums(wide[:, 32:32 + K], w), stack)
    # the norm adds the stack, in order, into the 32-bit stream
    for out_dtype in (torch.bfloat16, torch.float32):
        stream = torch.randn(M, N, device=DEV)
        gain = (1 + 0.2 * torch.randn(N)).to(DEV)
        total = stream.clone()
        for part in stack:
            total += part
        y = ops.add_rmsnorm(stack, stream, gain, 1e-5, out_dtype)
        assert torch.equal(stream, total)
        ref = plain.rms_norm(total.cpu(), gain.cpu(), 1e-5)
        assert (y.float().cpu() - ref).abs().max() <= tol(out_dtype, ref)
        rows = torch.tensor([M - 1, 0], dtype=torch.int32, device=DEV)          # selected rows: the stream stays
        y2 = ops.add_rmsnorm(stack, stream, gain, 1e-5, out_dtype, rows=rows)
        ref2 = plain.rms_norm((total + stack.sum(0)).cpu()[[M - 1, 0]], gain.cpu(), 1e-5)
        assert torch.equal(stream, total) and (y2.float().cpu() - ref2).abs().max() <= tol(out_dtype, ref2)


def test_gemm_dispatch_refuses_nothing_silently(ops):
    a = torch.randn(4, 20, device=DEV).bfloat16()          # K not a multiple of 8: the general kernel takes it
    w = torch.randn(6, 20, device=DEV).bfloat16()
    assert not ops.gemm_skinny_supports(a, w)
    got = ops.gemm_bf16(a, w, out_dtype=torch.float32)
    assert (got - a.float() @ w.float().T).abs().max() < 1e-4
    with pytest.raises(ops.KernelError):
        ops.gemm_skinny(a, w)
    # 32-bit results over very many columns (a logits head) at 17 to 32 rows, and just past them
    torch.manual_seed(18)
    w = (torch.randn(70001, 264, device=DEV) * 0.2).bfloat16()
    for M in (17, 32, 33):
        a = torch.randn(M, 264, device=DEV).bfloat16()
        got = ops.gemm_bf16(a, w, out_dtype=torch.float32)
        want = a.double().cpu() @ w.double().cpu().T
        assert got.dtype == torch.float32 and (got.double().cpu() - want).abs().max() <= 2e-5 * float(want.abs().max())


@pytest.mark.parametrize("shape", [(1, 48, 64), (8, 503, 96), (16, 256, 4096), (17, 100, 224), (40, 96, 1032),
                                   (64, 2100, 520), (5, 4096, 128)])
@pytest.mark.parametrize("nt", [0, 1, 2, 4])
def test_gemm_skinny_fused_forms(ops, shape, nt):
    """The folded forms against the separate kernels' references: the add into the 32-bit residual
    behind a product, and silu(gate) * up behind the product with the stacked gate|up weights."""
    torch.manual_seed(11)
    M, N, K = shape
    if nt == 4 and M <= 16:
        nt = 2
    w = (torch.randn(N, K, device=DEV) * 0.3).bfloat16()
    # add into the residual (whose rows must be 16-byte aligned)
    n4 = N - N % 4
    a = torch.randn(M, K, device=DEV).bfloat16()
    stream = torch.randn(M, n4, device=DEV)
    want = stream.cpu() + a.float().cpu() @ w[:n4].float().cpu().T
    ops.gemm_skinny_add(a, w[:n4], stream, nt=nt)
    assert (stream.cpu() - want).abs().max() <= 1e-4 * want.abs().max() + 1e-4
    # gate|up: any I, also one that is no multiple of 16 (N odd: drop a row so that the halves are equal)
    inter = N // 2
    if inter:
        wgu = torch.cat([w[:inter], w[N - inter:]]).contiguous()
        gate_up = a.float().cpu() @ wgu.float().cpu().T
        want = plain.silu_and_mul(gate_up)
        got = ops.gemm_skinny_silu(a, wgu, nt=nt if nt != 1 else 0)
        assert got.shape == (M, inter) and got.dtype == torch.bfloat16
        assert (got.float().cpu() - want).abs().max() <= 1e-2 * want.abs().max()


@pytest.mark.parametrize("shape", [(17, 520, 512), (33, 520, 1024), (64, 132, 2112), (40, 4100, 256), (5, 96, 4096),
                                   (64, 12288, 4096), (48, 6144, 4096), (24, 17408, 5120), (64, 100, 192),
                                   (65, 520, 512), (80, 12288, 1024), (96, 12288, 4096), (97, 4100, 256), (128, 17408, 5120),
                                   (113, 3072, 1024), (128, 9000, 640)])
def test_gemm_rows(ops, shape):
    """The product for 17 to 128 rows with its epilogues: plain, with bias, and silu(gate) * up on the stacked
    matrix; sizes that cut into whole tiles and sizes that do not, one and several groups of waves along K."""
    torch.manual_seed(21)
    M, N, K = shape
    x = torch.randn(M, K, device=DEV).bfloat16()
    w = (torch.randn(2 * N, K, device=DEV) * K ** -0.5).bfloat16()
    bias = torch.randn(N, device=DEV)
    y = x.float() @ w.float().T
    assert ops.gemm_rows_supports(x, w[:N])
    got = ops.gemm_rows(x, w[:N])
    assert got.dtype == torch.bfloat16 and (got.float() - y[:, :N]).abs().max() <= tol(torch.bfloat16, y[:, :N])
    got = ops.gemm_rows(x, w[:N], bias)
    assert (got.float() - (y[:, :N] + bias)).abs().max() <= tol(torch.bfloat16, y[:, :N] + bias)
    if M > 96 and N <= 8192:
        # 128 rows of X over the threads of two waves (at most 32 columns a block), and two tiles of W a wave:
        # refused, the caller takes the library
        assert not ops.gemm_rows_supports(x, w, silu=True)
    else:
        want = F.silu(y[:, :N]) * y[:, N:]
        got = ops.gemm_rows(x, w, silu=True)
        assert (got.float() - want).abs().max() <= tol(torch.bfloat16, want)
        # the same rows in another batch give the same bits: the cut of the matrix does not depend on the rows
        if M > 20:
            again = ops.gemm_rows(x[3:20].contiguous(), w, silu=True)
            assert torch.equal(again, got[3:20])
    with pytest.raises(ops.KernelError):
        ops.gemm_rows(torch.randn(129, K, device=DEV).bfloat16(), w[:N])

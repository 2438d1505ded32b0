"""Trace replay against the plain implementation: each request alone and whole; most of it in one
step and the last 32 tokens one by one; portions of changing size down to two tokens; mixed with up
to four live requests and so few pages that they are used again; long decoding; first tokens.
In 32-bit and in bfloat16, for three tiny configurations."""
import numpy as np
import pytest
import torch

import plain_qwen3 as plain
from gpu_util import DEV

pytestmark = pytest.mark.gpu

REL = {"float32": 2e-5, "bfloat16": 3e-2}


def close(got, want, dtype):
    want = want.numpy() if isinstance(want, torch.Tensor) else want
    bound = REL[dtype] * float(np.abs(want).max()) + 1e-6
    err = float(np.abs(got - want).max())
    assert err <= bound, f"max |diff| {err:.3e} > {bound:.3e}"


def make_tokens(vocab, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


@pytest.fixture(scope="module")
def replayers(model_dirs):
    from ullm_amd.replay import Replayer
    cache = {}

    def get(name, dtype, max_tokens=512, page_size=16):
        key = (name, dtype, max_tokens, page_size)
        if key not in cache:
            cache[key] = Replayer(model_dirs[name], dtype, max_tokens, page_size, DEV)
        rep = cache[key]
        assert not rep.live and rep.runner.cache.num_free_pages() == rep.max_tokens // page_size
        return rep
    return get


def oracle(plain_models, name, toks):
    cfg, w = plain_models[name]
    return plain.qwen3_forward(w, cfg, toks)


CASES = [(n, d) for n in ("A", "B", "C", "D", "E") for d in ("float32", "bfloat16")]


@pytest.mark.parametrize("name,dtype", CASES)
def test_whole(replayers, plain_models, name, dtype):
    rep = replayers(name, dtype)
    vocab = plain_models[name][0]["vocab_size"]
    for i, n in enumerate((1, 2, 17, 70, 113)):
        toks = make_tokens(vocab, n, 10 + i)
        got = rep.step({"step": i, "entries": [{"id": "r", "tokens": toks, "want": list(range(n))}], "end": ["r"]})
        close(got, oracle(plain_models, name, toks), dtype)


@pytest.mark.parametrize("name,dtype", CASES)
def test_bulk_then_one_by_one(replayers, plain_models, name, dtype):
    rep = replayers(name, dtype)
    vocab = plain_models[name][0]["vocab_size"]
    toks = make_tokens(vocab, 101, 20)
    want = oracle(plain_models, name, toks)
    head = len(toks) - 32
    got = [rep.step({"step": 0, "entries": [{"id": "r", "tokens": toks[:head], "want": [head - 1]}], "end": []})]
    for i in range(head, len(toks)):
        got.append(rep.step({"step": i, "entries": [{"id": "r", "tokens": [toks[i]], "want": [0]}],
                             "end": ["r"] if i == len(toks) - 1 else []}))
    close(np.concatenate(got), want[head - 1:], dtype)


@pytest.mark.parametrize("name,dtype", CASES)
def test_changing_portions(replayers, plain_models, name, dtype):
    rep = replayers(name, dtype)
    vocab = plain_models[name][0]["vocab_size"]
    toks = make_tokens(vocab, 150, 21)
    want = oracle(plain_models, name, toks)
    sizes = [2, 3, 16, 2, 15, 17, 1, 31, 2, 33, 5, 2, 2, 19]
    assert sum(sizes) == 150
    got, i = [], 0
    for s, n in enumerate(sizes):
        got.append(rep.step({"step": s, "entries": [{"id": "r", "tokens": toks[i:i + n], "want": list(range(n))}],
                             "end": ["r"] if i + n == 150 else []}))
        i += n
    close(np.concatenate(got), want, dtype)


@pytest.mark.parametrize("name,dtype", CASES)
def test_mixed_with_page_reuse(replayers, plain_models, name, dtype):
    """Seven requests, at most four live, portions of some beside decoded tokens of others.  The pool
    holds 256 tokens while the requests need 2.4 times that in total, so pages are used again."""
    rep = replayers(name, dtype, max_tokens=256, page_size=16)
    vocab = plain_models[name][0]["vocab_size"]
    lens = [70, 33, 90, 47, 61, 5, 64]
    reqs = {f"q{i}": make_tokens(vocab, n, 30 + i) for i, n in enumerate(lens)}
    wants = {r: oracle(plain_models, name, t) for r, t in reqs.items()}
    done = {r: 0 for r in reqs}
    got = {r: [] for r in reqs}
    waiting = list(reqs)
    live = []
    rng = np.random.default_rng(0)
    step = 0
    freed_pages = set()
    reused = False
    while waiting or live:
        while waiting and len(live) < 4:
            cand = waiting[0]
            held = sum(-(-max(done[r], 1) // 64) * 64 for r in live)
            if held + -(-len(reqs[cand]) // 64) * 64 > 256:
                break
            live.append(waiting.pop(0))
        entries, ends = [], []
        for r in list(live):
            rest = len(reqs[r]) - done[r]
            if done[r] >= len(reqs[r]) - 8:
                n = 1                                               # decode the tail token by token
            else:
                n = int(min(rest, rng.choice([2, 3, 7, 16, 29])))
            if rng.random() < 0.15 and len(live) > 1:
                continue                                            # left out of this step, goes on later
            entries.append({"id": r, "tokens": reqs[r][done[r]:done[r] + n], "want": list(range(n))})
            done[r] += n
            if done[r] == len(reqs[r]):
                ends.append(r)
                live.remove(r)
        for r in ends:                                              # pages about to be given back
            freed_pages |= set(rep.live[r].tables[0]) if r in rep.live else set()
        out = rep.step({"step": step, "entries": entries, "end": ends})
        for rc in rep.live.values():
            reused |= bool(freed_pages & {p for p in rc.tables[0] if p >= 0})
        row = 0
        for e in entries:
            n = len(e["tokens"])
            got[e["id"]].append(out[row:row + n])
            row += n
        step += 1
        rep.runner.cache.check()
    for r in reqs:
        close(np.concatenate(got[r]), wants[r], dtype)
    total_pages = sum(-(-n // 16) for n in lens)
    assert total_pages > 256 // 16                                  # more pages were needed than exist
    assert reused                                                   # a later request got a page an ended one had used


@pytest.mark.parametrize("name", ["B", "C"])
def test_portions_whose_projections_come_as_stacks_of_partial_sums(model_dirs, plain_models, name, monkeypatch):
    """Steps of 17 to 256 tokens hand the output and down projections to the next norm as stacks of
    partial sums where the matrices are large; here the size limit is lifted so that the tiny model
    takes that way too, beside steps that do not."""
    import dataclasses
    from ullm_amd.kernels import dispatch
    from ullm_amd.parts import linear
    from ullm_amd.replay import Replayer
    rules = dispatch.default_limits
    monkeypatch.setattr(dispatch, "default_limits", lambda c, k: dataclasses.replace(rules(c, k), stacked_from=17, stacked_to=256))
    calls, inner = [], linear.ops.gemm_partial_sums
    monkeypatch.setattr(linear.ops, "gemm_partial_sums", lambda x, w: calls.append(x.shape[0]) or inner(x, w))
    rep = Replayer(model_dirs[name], "bfloat16", 512, 16, DEV)
    vocab = plain_models[name][0]["vocab_size"]
    toks = make_tokens(vocab, 250, 31)
    want = oracle(plain_models, name, toks)
    sizes = [17, 3, 64, 40, 1, 60, 16, 25, 24]
    assert sum(sizes) == 250
    got, i = [], 0
    for s, n in enumerate(sizes):
        got.append(rep.step({"step": s, "entries": [{"id": "r", "tokens": toks[i:i + n], "want": list(range(n))}],
                             "end": ["r"] if i + n == 250 else []}))
        i += n
    assert set(calls) == {n for n in sizes if n >= 17}
    close(np.concatenate(got), want, "bfloat16")


def test_portions_of_17_to_64_tokens_through_the_kernel_for_those_row_counts(model_dirs, plain_models, monkeypatch):
    """Steps of 17 to 64 tokens take the q|k|v and gate|up projections through the kernel for those row counts where
    the matrices are large; here the size limit is lifted so that a tiny model (A: width 64, a whole stage of K)
    takes that way too, beside steps that do not."""
    import dataclasses
    from ullm_amd.kernels import dispatch, ops
    from ullm_amd.replay import Replayer
    rules = dispatch.default_limits
    monkeypatch.setattr(dispatch, "default_limits",
                        lambda c, k: dataclasses.replace(rules(c, k), rows=64, silu_skinny=16, silu_rows=64))
    calls, inner = [], ops.gemm_rows
    monkeypatch.setattr(ops, "gemm_rows", lambda a, w, bias=None, silu=False: calls.append((a.shape[0], silu)) or inner(a, w, bias, silu))
    rep = Replayer(model_dirs["A"], "bfloat16", 512, 16, DEV)
    vocab = plain_models["A"][0]["vocab_size"]
    toks = make_tokens(vocab, 250, 32)
    want = oracle(plain_models, "A", toks)
    sizes = [17, 3, 64, 40, 1, 60, 16, 25, 24]
    assert sum(sizes) == 250
    got, i = [], 0
    for s, n in enumerate(sizes):
        got.append(rep.step({"step": s, "entries": [{"id": "r", "tokens": toks[i:i + n], "want": list(range(n))}],
                             "end": ["r"] if i + n == 250 else []}))
        i += n
    assert {n for n, _ in calls} == {n for n in sizes if 17 <= n <= 64}
    assert {silu for _, silu in calls} == {False, True}               # q|k|v and gate|up
    close(np.concatenate(got), want, "bfloat16")


@pytest.mark.parametrize("name,dtype", [("B", "float32"), ("C", "bfloat16"), ("C", "float32"), ("D", "bfloat16"),
                                        ("E", "bfloat16")])
def test_long_decoding(replayers, plain_models, name, dtype):
    rep = replayers(name, dtype)
    vocab = plain_models[name][0]["vocab_size"]
    toks = make_tokens(vocab, 230, 40)
    want = oracle(plain_models, name, toks)
    got = [rep.step({"step": 0, "entries": [{"id": "r", "tokens": toks[:3], "want": [0, 1, 2]}], "end": []})]
    for i in range(3, len(toks)):
        got.append(rep.step({"step": i, "entries": [{"id": "r", "tokens": [toks[i]], "want": [0]}],
                             "end": ["r"] if i == len(toks) - 1 else []}))
    close(np.concatenate(got), want, dtype)


@pytest.mark.parametrize("name,dtype", CASES)
def test_first_tokens_and_skipped_logits(replayers, plain_models, name, dtype):
    rep = replayers(name, dtype)
    vocab = plain_models[name][0]["vocab_size"]
    toks = make_tokens(vocab, 20, 41)
    want = oracle(plain_models, name, toks)
    a = rep.step({"step": 0, "entries": [{"id": "r", "tokens": toks[:1], "want": [0]}], "end": []})
    close(a, want[:1], dtype)
    assert rep.step({"step": 1, "entries": [{"id": "r", "tokens": toks[1:9], "want": []}], "end": []}) is None
    b = rep.step({"step": 2, "entries": [{"id": "r", "tokens": toks[9:20], "want": [10, 0]}], "end": ["r"]})
    close(b, want[[19, 9]], dtype)                                   # order of `want` is kept


ODD_SIZES = [dict(hidden_size=90, num_attention_heads=3, num_key_value_heads=1, head_dim=16, intermediate_size=100,
                  vocab_size=301),                                  # a width that is no multiple of 4
             dict(hidden_size=36, num_attention_heads=2, num_key_value_heads=2, head_dim=80, intermediate_size=44,
                  vocab_size=77),                                   # heads wider than the model
             dict(hidden_size=100, num_attention_heads=4, num_key_value_heads=2, head_dim=112, intermediate_size=108,
                  vocab_size=130)]


@pytest.mark.parametrize("sizes", ODD_SIZES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sizes_the_vector_kernels_do_not_take(tmp_path, sizes, dtype):
    """Widths, head sizes and vocabularies that are no multiples of 8 (or of 4): the kernels with 16-byte
    accesses must step aside for the general ones, in a prompt portion and in one-token steps."""
    from ullm_amd.replay import Replayer
    from ullm_amd.weights.random_init import write_random_model
    cfg = dict(architectures=["Qwen3ForCausalLM"], num_hidden_layers=2, rope_theta=10000.0, rms_norm_eps=1e-5,
               max_position_embeddings=128, tie_word_embeddings=False, attention_bias=True, use_sliding_window=False,
               initializer_range=0.05, torch_dtype="bfloat16", **sizes)
    write_random_model(cfg, str(tmp_path), seed=3)
    pcfg, w = plain.load_model_folder(str(tmp_path))
    rep = Replayer(str(tmp_path), dtype, 256, 16, DEV)
    toks = make_tokens(cfg["vocab_size"], 60, 1)
    want = plain.qwen3_forward(w, pcfg, toks)
    got = [rep.step({"step": 0, "entries": [{"id": "r", "tokens": toks[:37], "want": list(range(37))}], "end": []})]
    for i in range(37, 60):
        got.append(rep.step({"step": i, "entries": [{"id": "r", "tokens": [toks[i]], "want": [0]}],
                             "end": ["r"] if i == 59 else []}))
    close(np.concatenate(got), want, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_long_context_beside_a_short_one(tmp_path, dtype):
    """2,600 tokens of one request (two long portions, then one token a step) beside a short request
    that decodes meanwhile: block tables of more than 1,024 keys, prompt tiles with many keys, decode
    steps whose keys are cut over many blocks."""
    from conftest import TINY_D
    from ullm_amd.replay import Replayer
    from ullm_amd.weights.random_init import write_random_model
    cfg = dict(TINY_D, max_position_embeddings=4096)
    write_random_model(cfg, str(tmp_path), seed=9)
    pcfg, w = plain.load_model_folder(str(tmp_path))
    rep = Replayer(str(tmp_path), dtype, 2816, 16, DEV)
    long, short = make_tokens(cfg["vocab_size"], 2600, 60), make_tokens(cfg["vocab_size"], 51, 61)
    wl, ws = plain.qwen3_forward(w, pcfg, long), plain.qwen3_forward(w, pcfg, short)
    got = rep.step({"step": 0, "entries": [{"id": "l", "tokens": long[:1500], "want": [0, 1499]},
                                           {"id": "s", "tokens": short[:20], "want": [19]}], "end": []})
    close(got, torch.stack([wl[0], wl[1499], ws[19]]), dtype)
    got = rep.step({"step": 1, "entries": [{"id": "s", "tokens": [short[20]], "want": [0]},
                                           {"id": "l", "tokens": long[1500:2570], "want": [0, 523, 524, 1069]}], "end": []})
    close(got, torch.stack([ws[20], wl[1500], wl[2023], wl[2024], wl[2569]]), dtype)
    for i in range(30):
        last = i == 29
        got = rep.step({"step": 2 + i, "entries": [{"id": "l", "tokens": [long[2570 + i]], "want": [0]},
                                                   {"id": "s", "tokens": [short[21 + i]], "want": [0]}], "end": ["l", "s"] if last else []})
        close(got, torch.stack([wl[2570 + i], ws[21 + i]]), dtype)


def test_other_page_sizes(replayers, plain_models):
    for page_size in (4, 64):
        rep = replayers("B", "float32", max_tokens=128, page_size=page_size)
        toks = make_tokens(503, 100, 42)
        want = oracle(plain_models, "B", toks)
        got = [rep.step({"step": 0, "entries": [{"id": "r", "tokens": toks[:61], "want": list(range(61))}], "end": []})]
        for i in range(61, 100):
            got.append(rep.step({"step": i, "entries": [{"id": "r", "tokens": [toks[i]], "want": [0]}],
                                 "end": ["r"] if i == 99 else []}))
        close(np.concatenate(got), want, "float32")


@pytest.mark.parametrize("trial,matrix_cores", [(t, False) for t in range(8)] + [(t, True) for t in range(8, 13)])
def test_random_configurations(tmp_path, trial, matrix_cores):
    """Configurations drawn at random over what config.json allows (head sizes in steps of 16, heads per
    kv head from 1 to 8, widths and vocabularies that are no powers of two, windows, tied heads, page
    sizes): portions of changing size and then single tokens equal the plain model, in both dtypes.
    With ``matrix_cores`` the head size and the page size are drawn among those the matrix-core attention
    kernels take, so that the bfloat16 run goes through them (the other trials mostly take the general kernel)."""
    import random
    from ullm_amd.kernels import ops
    from ullm_amd.replay import Replayer
    from ullm_amd.weights.random_init import write_random_model
    rng = random.Random(1000 + trial)
    nkv = rng.choice([1, 2, 3, 4, 8])
    cfg = dict(architectures=["Qwen3ForCausalLM"], hidden_size=rng.choice([40, 72, 96, 136, 200, 264]),
               num_hidden_layers=rng.choice([1, 2, 3]), num_attention_heads=nkv * rng.choice([1, 2, 3, 4, 5, 7, 8]),
               num_key_value_heads=nkv, head_dim=rng.choice([16, 32, 48, 64, 80, 96, 112, 128, 256]),
               intermediate_size=rng.choice([56, 104, 200, 328]), vocab_size=rng.choice([101, 257, 503, 1000]),
               rope_theta=rng.choice([1e4, 1e6]), rms_norm_eps=rng.choice([1e-5, 1e-6]), max_position_embeddings=512,
               tie_word_embeddings=rng.random() < 0.5, initializer_range=0.05, use_sliding_window=rng.random() < 0.4,
               sliding_window=rng.choice([7, 33, 100]), max_window_layers=rng.choice([0, 1]))
    page_size, n = rng.choice([4, 8, 16, 32]), rng.choice([40, 97, 150])
    if matrix_cores:
        cfg["head_dim"] = rng.choice([32, 64, 96, 128, 256])
        cfg["use_sliding_window"] = trial % 2 == 0
        page_size, n = rng.choice([16, 32, 64]), rng.choice([97, 150, 230])
    if cfg["use_sliding_window"] and trial % 3 == 0:          # the windowed layers named one by one
        cfg["layer_types"] = [rng.choice(["full_attention", "sliding_attention"]) for _ in range(cfg["num_hidden_layers"])]
    assert ops.attention_mfma_supports(torch.bfloat16, cfg["head_dim"], page_size, cfg["num_attention_heads"], nkv) == matrix_cores \
        or not matrix_cores
    d = write_random_model(cfg, str(tmp_path / "m"), seed=trial)
    pc, w = plain.load_model_folder(d)
    toks = [rng.randrange(cfg["vocab_size"]) for _ in range(n)]
    want = plain.qwen3_forward(w, pc, toks)
    cuts, left = [], n - 12
    while left > 0:
        cuts.append(min(left, rng.choice([2, 3, 17, 33, 64])))
        left -= cuts[-1]
    cuts += [1] * 12
    for dtype in ("float32", "bfloat16"):
        rep = Replayer(d, dtype, 512, page_size, DEV)
        outs, i = [], 0
        for s, c in enumerate(cuts):
            outs.append(rep.step({"step": s, "entries": [{"id": "a", "tokens": toks[i:i + c], "want": list(range(c))}],
                                  "end": []}))
            i += c
        close(np.concatenate(outs), want, dtype)


@pytest.mark.parametrize("trial", range(16))
def test_random_mixed_traces(tmp_path, trial):
    """Random configurations under random traces: up to four live requests in a pool that holds just them,
    each cut in its own manner (portions of changing size, most of it at once and then single tokens, single
    tokens from its middle on), some left out of a step; a request is admitted as soon as the pool has room,
    on pages that others gave back.  Every position's logits equal the plain model's, in both dtypes."""
    import random
    from ullm_amd.replay import Replayer
    from ullm_amd.weights.random_init import write_random_model
    rng = random.Random(5000 + trial)
    nkv = rng.choice([1, 2, 3, 4, 8])
    cfg = dict(architectures=["Qwen3ForCausalLM"], hidden_size=rng.choice([40, 72, 96, 136, 200, 264]),
               num_hidden_layers=rng.choice([1, 2, 3]), num_attention_heads=nkv * rng.choice([1, 2, 3, 4, 5, 7, 8]),
               num_key_value_heads=nkv, head_dim=rng.choice([16, 32, 48, 64, 80, 96, 112, 128, 256]),
               intermediate_size=rng.choice([56, 104, 200, 328]), vocab_size=rng.choice([101, 257, 503, 1000]),
               rope_theta=rng.choice([1e4, 1e6]), rms_norm_eps=rng.choice([1e-5, 1e-6]), max_position_embeddings=1024,
               tie_word_embeddings=rng.random() < 0.5, attention_bias=rng.random() < 0.3, initializer_range=0.05,
               use_sliding_window=rng.random() < 0.4, sliding_window=rng.choice([7, 33, 100, 150]),
               max_window_layers=rng.choice([0, 1]))
    page_size = rng.choice([4, 8, 16, 32])
    if trial % 2:                                             # shapes the matrix-core attention takes
        cfg["head_dim"], page_size = rng.choice([32, 64, 96, 128, 256]), rng.choice([16, 32, 64])
    d = write_random_model(cfg, str(tmp_path / "m"), seed=trial)
    pc, w = plain.load_model_folder(d)
    lens = [rng.choice([3, 20, 64, 65, 130, 257, 400]) for _ in range(rng.choice([2, 3, 4, 5, 6]))]
    toks = {f"r{i}": [rng.randrange(cfg["vocab_size"]) for _ in range(n)] for i, n in enumerate(lens)}
    want = {r: plain.qwen3_forward(w, pc, t).numpy() for r, t in toks.items()}
    held = lambda r: -(-len(toks[r]) // 64) * 64             # noqa: E731
    pool = max(sum(sorted((held(r) for r in toks), reverse=True)[:4]), 128)
    manner = {r: rng.choice(["portions", "most, then single", "single from the middle"]) for r in toks}
    steps, done, live, queue = [], {r: 0 for r in toks}, [], list(toks)
    while queue or live:
        while queue and len(live) < 4 and sum(held(x) for x in live) + held(queue[0]) <= pool:
            live.append(queue.pop(0))
        entries, end = [], []
        for r in [r for r in live if rng.random() < 0.8] or [live[0]]:
            left = len(toks[r]) - done[r]
            if manner[r] == "portions":
                n = min(left, rng.choice([1, 2, 3, 5, 17, 31, 32, 33, 64, 100]))
            elif manner[r] == "most, then single":
                n = left - 12 if left > 12 else 1
            else:
                n = min(left, rng.choice([2, 40])) if done[r] < len(toks[r]) // 2 else 1
            entries.append((r, done[r], n))
            done[r] += n
            if done[r] == len(toks[r]):
                end.append(r)
        steps.append((entries, end))
        live = [r for r in live if r not in end]
    for dtype in ("float32", "bfloat16"):
        rep = Replayer(d, dtype, pool, page_size, DEV)
        for s, (entries, end) in enumerate(steps):
            got = rep.step({"step": s, "end": end, "entries": [
                {"id": r, "tokens": toks[r][at:at + n], "want": list(range(n))} for r, at, n in entries]})
            row = 0
            for r, at, n in entries:
                bound = REL[dtype] * float(np.abs(want[r]).max()) + 1e-6
                err = float(np.abs(got[row:row + n] - want[r][at:at + n]).max())
                assert err <= bound, f"{dtype} step {s} request {r} tokens {at}..{at + n - 1}: {err:.3e} > {bound:.3e}"
                row += n
        assert not rep.live and rep.runner.cache.num_free_pages() == rep.max_tokens // page_size


def test_bfloat16_attention_off_the_matrix_cores_is_announced(model_dirs, caplog):
    """Head sizes and page sizes the matrix-core kernels do not take run on the general kernel: right, but
    many times slower, so it is said once per shape."""
    import logging
    from ullm_amd.kernels import ops
    from ullm_amd.replay import Replayer
    ops._warned_general_attention.clear()
    with caplog.at_level(logging.WARNING, logger="ullm_amd"):
        rep = Replayer(model_dirs["C"], "bfloat16", 128, 16, DEV)                 # head_dim 48
        for i in range(3):
            rep.step({"step": i, "entries": [{"id": "r", "tokens": [1, 2, 3], "want": []}], "end": []})
        rep = Replayer(model_dirs["D"], "bfloat16", 128, 8, DEV)                  # pages of 8
        rep.step({"step": 0, "entries": [{"id": "r", "tokens": [1, 2, 3], "want": []}], "end": []})
        rep = Replayer(model_dirs["D"], "bfloat16", 128, 16, DEV)                 # taken by the matrix cores: silent
        rep.step({"step": 0, "entries": [{"id": "r", "tokens": [1, 2, 3], "want": []}], "end": []})
        rep = Replayer(model_dirs["C"], "float32", 128, 16, DEV)                  # 32-bit never goes there: silent
        rep.step({"step": 0, "entries": [{"id": "r", "tokens": [1, 2, 3], "want": []}], "end": []})
    said = [r.getMessage() for r in caplog.records if "general kernel" in r.getMessage()]
    assert len(said) == 2 and "head_dim 48" in said[0] and "page size 8" in said[1]


def test_pool_too_small_is_an_error_not_a_wrong_result(replayers):
    rep = replayers("A", "float32", max_tokens=64)
    with pytest.raises(RuntimeError, match="pages"):
        rep.step({"step": 0, "entries": [{"id": "r", "tokens": list(range(65)), "want": []}], "end": []})
    rep.step({"step": 1, "entries": [], "end": ["r"]})


def test_trace_run_program(trace_run, model_dirs, plain_models):
    """The program itself: protocol on stdin/stdout, files in --out, exit code."""
    for dtype in ("float32", "bfloat16"):
        tr = trace_run(model_dirs["B"], dtype, 128)
        toks = make_tokens(503, 40, 43)
        want = oracle(plain_models, "B", toks)
        a = tr.step([("x", toks[:30], [29]), ("y", toks[:5], [])])
        b = tr.step([("x", toks[30:31], [0]), ("y", toks[5:40], [34, 0])], end=["y"])
        c = tr.step([("x", toks[31:40], list(range(9)))], end=["x"])
        tr.close()
        close(a, want[29:30], dtype)
        close(b, want[[30, 39, 5]], dtype)
        close(c, want[31:], dtype)


@pytest.mark.parametrize("name", ["B", "C", "D"])
def test_steps_of_few_tokens_hand_the_norms_from_product_to_product(model_dirs, plain_models, name, monkeypatch):
    """In a bfloat16 step of up to 16 tokens every product that ends in the stream prepares the norm behind it, so
    between the first layer's norm and the last one no norm kernel runs and no product takes 32-bit rows to fold a
    norm in; with the hand-over switched off the same step folds or runs a norm per part and gives the same logits
    up to rounding.  Both against the plain model."""
    from ullm_amd.kernels import ops
    from ullm_amd.parts.attention import GQAttention
    from ullm_amd.parts.feedforward import SwiGLU
    from ullm_amd.replay import Replayer
    cfg = plain_models[name][0]
    layers, vocab = cfg["num_hidden_layers"], cfg["vocab_size"]
    toks = make_tokens(vocab, 40, 77)
    want = oracle(plain_models, name, toks)
    calls, inner, inner_folded = [], ops.add_rmsnorm, ops.gemm_skinny_normed
    monkeypatch.setattr(ops, "add_rmsnorm", lambda *a, **k: calls.append(1) or inner(*a, **k))
    monkeypatch.setattr(ops, "gemm_skinny_normed", lambda *a, **k: calls.append(1) or inner_folded(*a, **k))
    results = {}
    for ahead in (True, False):
        monkeypatch.setattr(GQAttention, "hands_norm_ahead", ahead)
        monkeypatch.setattr(SwiGLU, "hands_norm_ahead", ahead)
        rep = Replayer(model_dirs[name], "bfloat16", 256, 16, DEV, use_graphs=False)
        rows = [rep.step({"step": 0, "entries": [{"id": "r", "tokens": toks[:24], "want": list(range(24))}], "end": []})]
        counts = []
        for i, n in enumerate((1, 7, 8)):                  # 24 + 1 + 7 + 8 = 40 tokens
            at = 24 + sum((1, 7, 8)[:i])
            calls.clear()
            rows.append(rep.step({"step": 1 + i, "entries": [{"id": "r", "tokens": toks[at:at + n], "want": list(range(n))}],
                                  "end": ["r"] if at + n == 40 else []}))
            counts.append(len(calls))
        results[ahead] = np.concatenate(rows)
        close(results[ahead], want, "bfloat16")
        if ahead:
            assert all(c == 2 for c in counts), counts      # the first layer's norm and the last
        else:
            assert all(c == 2 * layers + 1 for c in counts), counts
    close(results[True], results[False], "bfloat16")


@pytest.mark.parametrize("name,dtype", [("B", "float32"), ("B", "bfloat16"), ("C", "bfloat16")])
def test_graph_replays_equal_eager_steps(model_dirs, plain_models, name, dtype):
    """Decode steps replayed from HIP graphs: every replay is checked against the same step run
    eagerly by a second runner, with eager work (prompt portions, other batch sizes) between the
    replays, and against the plain implementation."""
    from ullm_amd.replay import Replayer
    graphs = Replayer(model_dirs[name], dtype, 512, 16, DEV, use_graphs=True)
    eager = Replayer(model_dirs[name], dtype, 512, 16, DEV, use_graphs=False)
    if not graphs.runner.use_graphs:
        pytest.skip("graphs need the GPU")
    vocab = plain_models[name][0]["vocab_size"]
    reqs = {r: make_tokens(vocab, n, 50 + i) for i, (r, n) in enumerate([("a", 60), ("b", 45), ("c", 80)])}
    wants = {r: oracle(plain_models, name, t) for r, t in reqs.items()}
    done = {r: 0 for r in reqs}
    got = {r: [] for r in reqs}
    plan = [[("a", 20), ("b", 30)], [("a", 1), ("b", 1)], [("a", 1), ("b", 1), ("c", 50)], [("a", 1), ("b", 1), ("c", 1)],
            [("a", 1), ("c", 1)], [("a", 7), ("c", 1)], [("a", 1), ("b", 1), ("c", 1)], [("a", 1)], [("a", 1), ("b", 1), ("c", 1)]]
    for i in range(12):
        plan.append([(r, 1) for r in reqs])
    for s, step in enumerate(plan):
        entries = []
        for r, n in step:
            n = min(n, len(reqs[r]) - done[r])
            if n > 0:
                # in some steps of single tokens one entry wants nothing: its row is then left out of the
                # replayed graph's logits on the device
                skip = s % 4 == 3 and r == "b" and all(m == 1 for _, m in step) and len(step) > 1
                entries.append({"id": r, "tokens": reqs[r][done[r]:done[r] + n], "want": [] if skip else list(range(n)),
                                "at": done[r]})
                done[r] += n
        if not entries:
            continue
        a = graphs.step({"step": s, "entries": entries, "end": []})
        b = eager.step({"step": s, "entries": entries, "end": []})
        close(a, b, dtype)
        row = 0
        for e in entries:
            n = len(e["want"])
            got[e["id"]].append((e["at"], a[row:row + n]))
            row += n
        assert row == len(a)
    assert len(graphs.runner._graphs) >= 2 and not eager.runner._graphs
    skipped = 0
    for r in reqs:
        for at, rows in got[r]:
            if len(rows):
                close(rows, wants[r][at:at + len(rows)], dtype)
            skipped += len(rows) == 0
    assert skipped >= 3

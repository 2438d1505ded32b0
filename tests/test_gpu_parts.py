"""Each part alone, parts in other arrangements than Qwen3's, and a toy mixer with state of its own
that is registered, built and stepped from outside the framework (tests/toy_arch.py)."""
import os

import numpy as np
import pytest
import torch

import plain_qwen3 as plain
import toy_arch
from gpu_util import DEV, tol

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]
REL = {"float32": 2e-5, "bfloat16": 3e-2}


def base_cfg(layers, **kw):
    cfg = dict(architectures=["ToyStackForCausalLM"], vocab_size=211, hidden_size=72, eps=2e-6, theta=3000.0,
               layers=layers, init_std=0.08)
    cfg.update(kw)
    return cfg


ATT = dict(mixer="attention", heads=6, kv_heads=3, head_dim=16, ffn_size=100)
TOY = dict(mixer="running_mean", ffn_size=60)


def run_and_compare(tmp_path, cfg, dtype, cuts, n_tokens=75, page_size=8, seed=11):
    """Write the toy model, replay one request in the given cuts beside a second request, compare
    every position with the toy architecture's plain forward."""
    from ullm_amd.replay import Replayer
    from ullm_amd.weights.random_init import write_random_model
    from safetensors.torch import load_file
    d = write_random_model(cfg, str(tmp_path / f"m{seed}"), seed=seed)
    w = load_file(os.path.join(d, "model.safetensors"))
    g = torch.Generator().manual_seed(seed)
    toks = torch.randint(0, cfg["vocab_size"], (n_tokens,), generator=g).tolist()
    other = torch.randint(0, cfg["vocab_size"], (40,), generator=g).tolist()
    want, want_other = toy_arch.toy_forward(w, cfg, toks), toy_arch.toy_forward(w, cfg, other)
    rep = Replayer(d, dtype, 256, page_size, DEV)
    got, got_other, i, j = [], [], 0, 0
    assert sum(cuts) == n_tokens
    for s, n in enumerate(cuts):
        entries = [{"id": "a", "tokens": toks[i:i + n], "want": list(range(n))}]
        m = min(7, len(other) - j)
        if m > 0:
            entries.insert(0, {"id": "b", "tokens": other[j:j + m], "want": list(range(m))})
        out = rep.step({"step": s, "entries": entries, "end": []})
        if m > 0:
            got_other.append(out[:m])
            out = out[m:]
            j += m
        got.append(out)
        i += n
    rep.step({"step": 999, "entries": [], "end": ["a", "b"]})
    rep.runner.cache.check()
    for g_, w_ in ((np.concatenate(got), want), (np.concatenate(got_other), want_other[:j])):
        bound = REL[dtype] * float(w_.abs().max()) + 1e-6
        assert float(np.abs(g_ - w_.numpy()).max()) <= bound
    return rep, w


CUTS = [75], [43] + [1] * 32, [2, 9, 1, 17, 2, 30, 3, 11]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("cuts", CUTS)
def test_toy_mixer_with_state_registers_builds_and_steps(tmp_path, dtype, cuts):
    """Layers 0 and 2 are attention, layer 1 is the toy mixer: different mixers in one model, state
    carried across portion boundaries, zeroed when a slot is taken again."""
    cfg = base_cfg([ATT, TOY, dict(ATT, heads=4, kv_heads=1, head_dim=32)])
    rep, w = run_and_compare(tmp_path, cfg, dtype, cuts)
    groups = rep.runner.cache.groups
    assert len(groups) == 2 and any(c.state is not None for c in rep.runner.caches.values())
    # the slots are used again by new requests: their state must start from zero
    toks = list(range(3, 30))
    out = rep.step({"step": 0, "entries": [{"id": "z", "tokens": toks, "want": [len(toks) - 1]}], "end": ["z"]})
    want = toy_arch.toy_forward(w, cfg, toks)[-1:]
    assert float(np.abs(out - want.numpy()).max()) <= REL[dtype] * float(want.abs().max()) + 1e-6


KEYS = dict(mixer="keys_only", dim=24, ffn_size=60)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("cuts", CUTS)
def test_toy_mixer_that_keeps_one_row_per_token_and_plans_its_own_work(tmp_path, dtype, cuts):
    """A mixer defined in the tests that keeps keys only (one float32 row per token, no values) and takes its
    work list from a planner of its own: the step function allocates the one pool it declares, runs its planner
    beside the attention kernels' and hands it the result, with no change to the framework's files.  Layer 3
    reads the cache layer 1 wrote."""
    cfg = base_cfg([ATT, KEYS, dict(KEYS, dim=40), KEYS], run_order=[[0, 0], [1, 1], [2, 2], [3, 1]])
    rep, _ = run_and_compare(tmp_path, cfg, dtype, cuts, seed=19)
    runner = rep.runner
    assert sorted(runner._planners) == ["attention", "toy_spans"]
    assert [(g.head_dim, g.rows) for g in runner.cache.groups] == [(16, None), (24, ((1, 24, 4),)), (40, ((1, 40, 4),))]
    for cache_id, dim in ((1, 24), (2, 40)):
        view = runner.caches[cache_id]
        assert sorted(view.pools) == ["latent"] and view.k_pool is None and view.v_pool is None
        assert view.pools["latent"].dtype == torch.float32 and view.pools["latent"].shape[1:] == (1, 8, dim)
    attention = runner.caches[0]
    assert sorted(attention.pools) == ["k", "v"] and attention.k_pool is attention.pools["k"]
    pages = runner.cache.allocators[0].num_pages
    item = 4 if dtype == "float32" else 2
    assert runner.cache_bytes() == pages * 8 * (2 * 3 * 16 * item + 24 * 4 + 40 * 4)
    assert runner.cache.groups[1].bytes_per_token(item) == 24 * 4


@pytest.mark.parametrize("dtype", DTYPES)
def test_state_mixer_steps_replayed_from_graphs(tmp_path, dtype):
    """A state mixer that says its single-token step can be captured keeps the model on HIP graphs:
    three requests (a batch padded to four, the padding entries' state going to the spare row) decode
    side by side from graphs, a fourth joins and one leaves on the way, and every step equals the plain
    forward: the state moves on once per step, also in the step that captures a graph."""
    from ullm_amd.replay import Replayer
    from ullm_amd.weights.random_init import write_random_model
    from safetensors.torch import load_file
    cfg = base_cfg([ATT, TOY, dict(ATT, heads=4, kv_heads=1, head_dim=32), TOY])
    d = write_random_model(cfg, str(tmp_path / "m"), seed=21)
    w = load_file(os.path.join(d, "model.safetensors"))
    rep = Replayer(d, dtype, 512, 8, DEV, use_graphs=True)
    if not rep.runner.use_graphs:
        pytest.skip("graphs need the GPU")
    g = torch.Generator().manual_seed(5)
    reqs = {r: torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist() for r, n in (("a", 40), ("b", 33), ("c", 47), ("d", 30))}
    wants = {r: toy_arch.toy_forward(w, cfg, t).numpy() for r, t in reqs.items()}
    done = {r: 0 for r in reqs}
    plan = [[("a", 12), ("b", 9), ("c", 20)]] + [[("a", 1), ("b", 1), ("c", 1)]] * 6 + [[("d", 11)]] + \
           [[("a", 1), ("b", 1), ("c", 1), ("d", 1)]] * 5 + [[("a", 1), ("c", 1), ("d", 1)]] * 8 + [[("c", 1)]] * 3
    ended = set()
    for s, step in enumerate(plan):
        entries = []
        for r, n in step:
            n = min(n, len(reqs[r]) - done[r])
            if n > 0:
                entries.append({"id": r, "tokens": reqs[r][done[r]:done[r] + n], "want": list(range(n))})
        end = ["b"] if s == 13 and "b" not in ended else []
        ended.update(end)
        out = rep.step({"step": s, "entries": entries, "end": end})
        row = 0
        for e in entries:
            n = len(e["tokens"])
            want = wants[e["id"]][done[e["id"]]:done[e["id"]] + n]
            assert float(np.abs(out[row:row + n] - want).max()) <= REL[dtype] * float(np.abs(want).max()) + 1e-6, (s, e["id"])
            done[e["id"]] += n
            row += n
    assert len(rep.runner._graphs) >= 2          # batches of 4 (3 padded, and 4) and of 1


@pytest.mark.parametrize("dtype", DTYPES)
def test_scaled_embedding_head_bias_and_capped_logits(tmp_path, dtype):
    """What a plan may say about the two ends of the model: the token rows scaled on their way into the
    stream, a bias on the logits, and a soft cap on them (tight enough here to bend the largest logits)."""
    cfg = base_cfg([ATT, dict(ATT, heads=4, kv_heads=2, head_dim=32)], embed_scale=72 ** 0.5, head_bias=True, logit_cap=3.0)
    rep, w = run_and_compare(tmp_path, cfg, dtype, CUTS[2], seed=13)
    assert "head.bias" in w and float(w["head.bias"].abs().max()) > 0
    cfg = base_cfg([ATT], tie=True, embed_scale=0.5, logit_cap=50.0)
    run_and_compare(tmp_path, cfg, dtype, CUTS[1], seed=14)


@pytest.mark.parametrize("dtype", DTYPES)
def test_only_state_layers_need_no_pages(tmp_path, dtype):
    cfg = base_cfg([TOY, TOY], tie=True)
    rep, _ = run_and_compare(tmp_path, cfg, dtype, CUTS[2])
    assert rep.runner.cache.groups == []


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("variant", [
    dict(rope="adjacent"), dict(rope="none"), dict(rope="half", rotary_dim=8), dict(qk_norm=False),
    dict(bias=True), dict(window=9), dict(scale=0.31), dict(heads=5, kv_heads=5, head_dim=48),
    dict(heads=8, kv_heads=1, head_dim=64)])
def test_attention_part_options(tmp_path, dtype, variant):
    """The attention mixer with another position encoding (adjacent pairs, partial rotation, none),
    without its norms, with biases, with a window, with a scale of its own, with other head shapes."""
    cfg = base_cfg([dict(ATT, **variant), ATT])
    run_and_compare(tmp_path, cfg, dtype, CUTS[2], seed=12)


@pytest.mark.parametrize("cuts", CUTS)
def test_toy_feed_forward_with_routing(tmp_path, cuts):
    """A feed-forward defined here that sends every token to one of three experts, in one layer of
    a model whose other layer is dense.  In 32-bit only: the choice of the expert is discontinuous,
    and in bfloat16 a near-tie of two router scores may go the other way, which is no fault."""
    cfg = base_cfg([dict(ATT, experts=3, ffn_size=40), ATT, dict(TOY, experts=2, ffn_size=24)])
    rep, _ = run_and_compare(tmp_path, cfg, "float32", cuts, seed=14)
    from ullm_amd.parts import registered_parts
    assert "toy_top1_experts" in registered_parts("ffn")


@pytest.mark.parametrize("dtype", DTYPES)
def test_toy_position_encoding_with_its_own_angles(tmp_path, dtype):
    """A position encoding defined here (angles linear in the pair index, adjacent pairs) handed to
    the framework's attention mixer: only its table is new."""
    cfg = base_cfg([dict(ATT, rope="toy_linear", angle_step=0.013), dict(ATT, rope="toy_linear", angle_step=0.4, heads=2,
                                                                         kv_heads=2, head_dim=32)])
    run_and_compare(tmp_path, cfg, dtype, CUTS[2], seed=15)
    from ullm_amd.parts import registered_parts
    assert "toy_linear_angles" in registered_parts("position")


@pytest.mark.parametrize("dtype", DTYPES)
def test_run_order_names_a_layer_twice_and_shares_a_cache(tmp_path, dtype):
    # layer 1 runs twice with a cache of its own each time; layer 2 reads the cache layer 0 wrote
    cfg = base_cfg([ATT, dict(ATT, window=13), ATT], run_order=[[0, 0], [1, 1], [1, 7], [2, 0]])
    rep, _ = run_and_compare(tmp_path, cfg, dtype, CUTS[2], seed=13)
    assert sorted(rep.runner.caches) == [0, 1, 7]
    _, model = __import__("ullm_amd.models", fromlist=["build_model"]).build_model(cfg)
    groups, cache_group, _ = model.cache_layout()
    assert {g.window: g.layers for g in groups} == {0: ((0, 0),), 13: ((1, 0), (7, 0))}


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_block_that_keeps_keys_and_values_and_state(tmp_path, dtype):
    """One block with two mixers, one with a paged cache (windowed) and one with fixed-size state: the
    block declares a list of needs and gets one view per need; an ordinary attention layer runs beside it."""
    cfg = base_cfg([dict(ATT, mixer="both", window=19), ATT, dict(TOY)])
    rep, _ = run_and_compare(tmp_path, cfg, dtype, CUTS[2], seed=17)
    model = rep.model
    groups, cache_group, states = model.cache_layout()
    assert {g.window: g.layers for g in groups} == {19: ((0, 0),), 0: ((1, 0),)}
    assert sorted(states) == [(0, 1), (2, 0)]
    both = rep.runner.caches[0]
    assert len(both.parts) == 2 and both.parts[0].k_pool is not None and both.parts[1].state is not None
    assert both.k_pool is both.parts[0].k_pool and both.state is both.parts[1].state
    assert rep.runner.caches[1].parts == [] and rep.runner.caches[2].state is not None


def test_parts_are_found_by_name_and_unknown_names_fail():
    from ullm_amd.parts import build_part, registered_parts
    assert "toy_running_mean" in registered_parts("mixer") and "gqa_attention" in registered_parts("mixer")
    assert "toy_keys_only" in registered_parts("mixer")
    assert "swiglu" in registered_parts("ffn") and registered_parts("block") == ["prenorm", "toy_two_mixers"]
    with pytest.raises(KeyError, match="no mixer part named"):
        build_part("mixer", "does_not_exist")
    with pytest.raises(ValueError, match="needs differ"):
        cfg = base_cfg([ATT, dict(ATT, window=5)], run_order=[[0, 0], [1, 0]])
        from ullm_amd.models import build_model
        build_model(cfg)[1].cache_layout()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_part_and_block_wiring(dtype):
    """The norm part alone: the pending branch is added into the 32-bit stream, then normalised."""
    from ullm_amd.parts import PartEnv, build_part
    env = PartEnv(torch.device(DEV), dtype, 16)
    norm = build_part("norm", "rmsnorm", size=40, eps=1e-4, weight_name="g")
    gain = 1 + 0.3 * torch.randn(40)
    norm.bind({"g": gain.to(DEV)}, env)
    res, br = torch.randn(6, 40), torch.randn(6, 40).to(dtype)
    stream = res.clone().to(DEV)
    y = norm.add_norm(br.to(DEV), stream, out_dtype=dtype)
    s = res + br.float()
    assert torch.equal(stream.cpu(), s)
    want = plain.rms_norm(s, gain, 1e-4)
    assert (y.float().cpu() - want).abs().max() <= tol(dtype, want)


def test_feed_forward_hands_the_norm_a_stack_of_partial_sums(monkeypatch):
    """For 17 to 256 rows in bfloat16 (its down projection has few long rows) the last projection of a feed-forward comes as a stack of float32
    partial sums if every norm of the model adds stacks; the norm's sum is the plain result."""
    from types import SimpleNamespace
    import dataclasses
    from ullm_amd.kernels import dispatch
    from ullm_amd.parts import PartEnv, build_part
    from ullm_amd.weights.loader import bind_tensors
    rules = dispatch.default_limits                           # the test's matrices are small: as if they were large
    monkeypatch.setattr(dispatch, "default_limits", lambda c, k: dataclasses.replace(rules(c, k), stacked_from=17, stacked_to=256))
    torch.manual_seed(5)
    H, I = 96, 224
    env = PartEnv(torch.device(DEV), torch.bfloat16, 16)
    ffn = build_part("ffn", "swiglu", hidden_size=H, intermediate_size=I, prefix="f")
    w = {f"f.{n}.weight": (torch.randn(*shape) * 0.1).bfloat16().to(DEV)
         for n, shape in (("gate_proj", (I, H)), ("up_proj", (I, H)), ("down_proj", (H, I)))}
    bind_tensors(ffn, w, env)
    norm = build_part("norm", "rmsnorm", size=H, eps=1e-5, weight_name="g")
    norm.bind({"g": torch.ones(H, device=DEV)}, env)
    assert norm.adds_stacks
    for T, stacked in ((40, True), (16, False), (200, True), (257, False)):
        x = torch.randn(T, H).bfloat16().to(DEV)
        plain_out = ffn.forward(x, SimpleNamespace(stacked_branches=False, dtype=torch.bfloat16))
        out = ffn.forward(x, SimpleNamespace(stacked_branches=True, dtype=torch.bfloat16))
        assert (out.dim() == 3) == stacked and plain_out.dim() == 2
        a, b = torch.zeros(T, H, device=DEV), torch.zeros(T, H, device=DEV)
        ya = norm.add_norm(out, a, out_dtype=torch.bfloat16)
        yb = norm.add_norm(plain_out, b, out_dtype=torch.bfloat16)
        assert (a - b).abs().max() <= 1e-2 * b.abs().max()        # the plain result is rounded to bfloat16, the stack is not
        assert (ya.float() - yb.float()).abs().max() <= 3e-2 * yb.float().abs().max()


def test_norm_left_to_the_feed_forwards_first_projection(monkeypatch):
    """With few rows and nothing left to add, the block hands a part that folds norms the norm as a
    record; the feed-forward then adds ffn(norm(stream)) into the stream, as the plain functions do.
    The rows' sizes differ by orders of magnitude, so that a scale from the wrong row shows."""
    from types import SimpleNamespace
    from ullm_amd.parts import PartEnv, PendingNorm, build_part
    from ullm_amd.parts.block import PreNormBlock
    from ullm_amd.weights.loader import bind_tensors
    torch.manual_seed(6)
    H, I, eps = 96, 224, 1e-3
    env = PartEnv(torch.device(DEV), torch.bfloat16, 16)
    ffn = build_part("ffn", "swiglu", hidden_size=H, intermediate_size=I, prefix="f")
    w = {f"f.{n}.weight": (torch.randn(*shape) * 0.1).bfloat16() for n, shape in
         (("gate_proj", (I, H)), ("up_proj", (I, H)), ("down_proj", (H, I)))}
    bind_tensors(ffn, w, env)
    gain = 1 + 0.3 * torch.randn(H)
    norm = build_part("norm", "rmsnorm", size=H, eps=eps, weight_name="g")
    norm.bind({"g": gain.to(DEV)}, env)
    ctx = SimpleNamespace(stacked_branches=False, dtype=torch.bfloat16)
    assert ffn.folds_norm
    from ullm_amd.kernels import ops
    seen, inner = [], ops.gemm_skinny_normed
    monkeypatch.setattr(ops, "gemm_skinny_normed", lambda *a, **k: seen.append(1) or inner(*a, **k))
    # a small matrix keeps the norm inside for every row count the kernel takes, a large one up to 8 rows
    import dataclasses
    from ullm_amd.kernels import dispatch
    rules = dispatch.default_limits
    cases = [(T, True, None) for T in (1, 7, 8, 9, 16)] + [(T, T <= 8, 0) for T in (8, 9, 16)]
    for T, folded, small in cases:
        if small is not None:
            monkeypatch.setattr(dispatch, "default_limits", lambda c, k: dataclasses.replace(rules(c, k), fold_norm=8))
        stream = torch.randn(T, H) * torch.logspace(-2, 2, T)[:, None]
        want = stream + plain.qwen3_mlp(plain.rms_norm(stream, gain, eps), {k: v.float() for k, v in w.items()}, "f")
        got = stream.clone().to(DEV)
        assert ffn.fusable(got, ctx)
        x = PreNormBlock._normed(norm, ffn, None, got, ctx)
        assert isinstance(x, PendingNorm)
        seen.clear()
        ffn.forward_fused(x, got, ctx)
        assert bool(seen) == folded
        assert (got.cpu() - want).abs().max() <= 2e-2 * (want - stream).abs().max()
    # something left to add: the norm runs as a kernel of its own
    x = PreNormBlock._normed(norm, ffn, torch.zeros(4, H, device=DEV, dtype=torch.bfloat16), torch.randn(4, H, device=DEV), ctx)
    assert isinstance(x, torch.Tensor)


def test_a_feed_forward_prepares_the_norm_that_follows_it(monkeypatch):
    """Told which norm comes next, the feed-forward's last kernel leaves that norm half done (the stream times the
    gain, the rows' sums of squares) and returns its record; a second feed-forward behind that norm takes the
    record, and no norm kernel runs in between.  Two feed-forwards in a row against the plain functions, with
    rows whose sizes differ by orders of magnitude; and the record is only taken for the norm it was made for."""
    from types import SimpleNamespace
    from ullm_amd.kernels import ops
    from ullm_amd.parts import PartEnv, PendingNorm, build_part
    from ullm_amd.parts.block import PreNormBlock
    from ullm_amd.weights.loader import bind_tensors
    torch.manual_seed(8)
    H, I, eps = 104, 232, 1e-3
    env = PartEnv(torch.device(DEV), torch.bfloat16, 16)
    ffns, ws, norms, gains = [], [], [], []
    for i in range(2):
        ffn = build_part("ffn", "swiglu", hidden_size=H, intermediate_size=I, prefix=f"f{i}")
        w = {f"f{i}.{n}.weight": (torch.randn(*shape) * 0.1).bfloat16() for n, shape in
             (("gate_proj", (I, H)), ("up_proj", (I, H)), ("down_proj", (H, I)))}
        bind_tensors(ffn, w, env)
        gain = 1 + 0.3 * torch.randn(H)
        norm = build_part("norm", "rmsnorm", size=H, eps=eps, weight_name="g")
        norm.bind({"g": gain.to(DEV)}, env)
        ffns.append(ffn), ws.append(w), norms.append(norm), gains.append(gain)
    ctx = SimpleNamespace(stacked_branches=False, dtype=torch.bfloat16)
    assert ffns[0].hands_norm_ahead
    norm_kernels, inner = [], ops.add_rmsnorm
    monkeypatch.setattr(ops, "add_rmsnorm", lambda *a, **k: norm_kernels.append(1) or inner(*a, **k))
    for T in (1, 5, 8, 9, 16):
        stream = torch.randn(T, H) * torch.logspace(-2, 2, T)[:, None]
        mid = stream + plain.qwen3_mlp(plain.rms_norm(stream, gains[0], eps), {k: v.float() for k, v in ws[0].items()}, "f0")
        want = mid + plain.qwen3_mlp(plain.rms_norm(mid, gains[1], eps), {k: v.float() for k, v in ws[1].items()}, "f1")
        got = stream.clone().to(DEV)
        x = PreNormBlock._normed(norms[0], ffns[0], None, got, ctx)
        record = ffns[0].forward_fused(x, got, ctx, then=norms[1])
        assert isinstance(record, PendingNorm) and record.norm is norms[1] and record.scaled is not None
        assert (got.cpu() - mid).abs().max() <= 2e-2 * (mid - stream).abs().max()
        norm_kernels.clear()
        x = PreNormBlock._normed(norms[1], ffns[1], record, got, ctx)
        assert x is record
        assert ffns[1].forward_fused(x, got, ctx) is None                 # told of no norm: nothing prepared
        assert not norm_kernels
        assert (got.cpu() - want).abs().max() <= 2e-2 * (want - stream).abs().max()
        # a record made for another norm is not taken: the block's own norm runs on the finished stream
        x = PreNormBlock._normed(norms[0], ffns[1], record, got, ctx)
        assert x is not record and isinstance(x, PendingNorm) and x.norm is norms[0] and x.scaled is None
        # a part that wants its input computed gets the normed stream
        x = PreNormBlock._normed(norms[1], None, record, got, ctx)
        assert isinstance(x, torch.Tensor) and norm_kernels
        assert (x.float().cpu() - plain.rms_norm(got.cpu(), gains[1], eps)).abs().max() <= 1e-2 * x.float().abs().max()
    # beyond the rows the kernels take, nothing is prepared
    big = torch.randn(40, H, device=DEV)
    assert not ffns[0].fusable(big, ctx)


def test_rotary_part_table_matches_the_plain_angles():
    from ullm_amd.parts import PartEnv, build_part
    rot = build_part("position", "rotary", head_dim=24, theta=777.0, rotary_dim=12, pairing="half")
    rot.bind({}, PartEnv(torch.device(DEV), torch.float32, 50))
    table, dim, style = rot.kernel_args()
    cos, sin = plain.rope_cos_sin(torch.arange(50), 12, 777.0)
    assert (dim, style) == (12, 1) and table.shape == (50, 12)
    assert torch.allclose(table.cpu(), torch.cat((cos, sin), -1), atol=1e-6)
    with pytest.raises(ValueError):
        build_part("position", "rotary", head_dim=24, theta=1.0, rotary_dim=13)

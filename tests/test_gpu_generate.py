"""Generation through the entry point: greedy tokens equal the plain implementation's; seeded
temperature sampling equals the plain sampler run on the engine's own logits; finish rules;
preemption and recomputation give the same tokens; the command line."""
import json
import os

import pytest
import torch

import plain_qwen3 as plain
from gpu_util import DEV

pytestmark = pytest.mark.gpu


def make_llm(model_dir, **kw):
    from ullm_amd import LLM, EngineConfig
    args = dict(model=model_dir, dtype="float32", max_bs=8, context_len=128, page_size=16, num_pages=64, device=DEV)
    args.update(kw)
    return LLM(EngineConfig(**args))


def prompts_of(vocab, lens, seed):
    g = torch.Generator().manual_seed(seed)
    return [torch.randint(0, vocab, (n,), generator=g).tolist() for n in lens]


@pytest.mark.parametrize("name,page_size,budget,chunk", [("A", 16, 64, 64), ("A", 16, 9, 4), ("B", 4, 16, 7),
                                                          ("C", 8, 12, 5), ("D", 16, 20, 9)])
def test_greedy_generation_equals_the_plain_implementation(model_dirs, plain_models, name, page_size, budget, chunk):
    from ullm_amd import SamplingParams
    cfg, w = plain_models[name]
    prompts = prompts_of(cfg["vocab_size"], (5, 11, 17, 1), 1)
    llm = make_llm(model_dirs[name], page_size=page_size, max_num_batched_tokens=budget, max_prefill_chunk=chunk)
    outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=8, ignore_eos=True))
    for p, o in zip(prompts, outs):
        assert o.token_ids == plain.greedy_generate(w, cfg, p, 8)
        assert o.finish_reason.name == "LENGTH" and o.num_prompt_tokens == len(p)
    llm.engine.runner.cache.check()
    assert llm.engine.runner.cache.num_free_pages() == 64


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_seeded_sampling_equals_the_plain_sampler_on_the_engines_logits(model_dirs, plain_models, dtype):
    """Config B's workload: prompts of 1, 3, 9, 33 and 70 tokens, temperature 0.7, 12 new tokens each,
    prompt portions of 7 with decodes beside them."""
    from ullm_amd import SamplingParams
    cfg, w = plain_models["B"]
    prompts = prompts_of(503, (1, 3, 9, 33, 70), 3)
    llm = make_llm(model_dirs["B"], dtype=dtype, page_size=4, num_pages=128, max_num_batched_tokens=24,
                   max_prefill_chunk=7)
    seen = {}

    def hook(sampling, logits):
        for s, row in zip(sampling, logits.float().cpu()):
            seen.setdefault(s.request.request_id, []).append((s.request.num_tokens, row))
    llm.engine.on_logits = hook
    params = [SamplingParams(temperature=0.7, top_k=50 if i % 2 else -1, top_p=0.9 if i == 2 else 1.0,
                             max_new_tokens=12, ignore_eos=True, seed=100 + i) for i in range(5)]
    ids = [f"s{i}" for i in range(5)]
    outs = llm.generate(prompts, params, ids)
    for i, (p, o) in enumerate(zip(prompts, outs)):
        assert len(o.token_ids) == 12
        for (pos, row), tok in zip(seen[ids[i]], o.token_ids):
            # the kernel sums in 32-bit: a draw within rounding of a CDF boundary may fall on either side
            assert tok in plain.sample_token_set(row, 0.7, params[i].top_k, params[i].top_p, 0.0, 100 + i, pos)
        # and the logits the engine sampled from are the plain implementation's
        full = plain.qwen3_forward(w, cfg, p + o.token_ids)
        for (pos, row) in seen[ids[i]]:
            bound = (2e-5 if dtype == "float32" else 3e-2) * float(full.abs().max()) + 1e-6
            assert float((row - full[pos - 1]).abs().max()) <= bound
    # The same seeds give the same tokens in another batch composition.  In 32-bit every kernel sums in
    # an order that does not depend on the batch, so the logits are the same bit for bit; in bfloat16 the
    # logits may differ by rounding between compositions, which can move a draw that lies on a boundary.
    if dtype == "float32":
        again = llm.generate(prompts[::-1], params[::-1])
        assert [o.token_ids for o in again[::-1]] == [o.token_ids for o in outs]


def test_preempted_requests_are_recomputed_to_the_same_tokens(model_dirs, plain_models):
    from ullm_amd import SamplingParams
    cfg, w = plain_models["B"]
    prompts = prompts_of(503, (20, 22, 18), 5)
    roomy = make_llm(model_dirs["B"], page_size=4, num_pages=128)
    want = [o.token_ids for o in roomy.generate(prompts, SamplingParams(temperature=0.8, max_new_tokens=20,
                                                                        ignore_eos=True, seed=7))]
    tight = make_llm(model_dirs["B"], page_size=4, num_pages=22)       # 88 tokens for 3 x ~40
    outs = tight.generate(prompts, SamplingParams(temperature=0.8, max_new_tokens=20, ignore_eos=True, seed=7))
    assert [o.token_ids for o in outs] == want
    assert tight.engine.scheduler.num_preemptions > 0 and roomy.engine.scheduler.num_preemptions == 0
    assert tight.engine.runner.cache.num_free_pages() == 22
    tight.engine.runner.cache.check()


def test_finish_rules_and_abort(model_dirs, plain_models):
    from ullm_amd import FinishReason, SamplingParams
    cfg, w = plain_models["B"]
    prompt = prompts_of(503, (6,), 8)[0]
    greedy = plain.greedy_generate(w, cfg, prompt, 6)
    llm = make_llm(model_dirs["B"], context_len=16)
    # eos: stops at the first generated token equal to eos_token_id, which is emitted (ullm/core/engine.py:177-181)
    out = llm.generate(prompt, SamplingParams(temperature=0.0, eos_token_id=greedy[2], max_new_tokens=6))
    stop_at = greedy.index(greedy[2])
    assert out.token_ids == greedy[:stop_at + 1] and out.finish_reason is FinishReason.STOP
    # max_tokens caps prompt + generated (engine.py:184-189)
    out = llm.generate(prompt, SamplingParams(temperature=0.0, max_tokens=9, ignore_eos=True))
    assert len(out.token_ids) == 3 and out.finish_reason is FinishReason.LENGTH
    # context_len caps the total (engine.py:196-198); a longer prompt keeps its last context_len tokens (:81-82)
    out = llm.generate(prompt, SamplingParams(temperature=0.0, ignore_eos=True))
    assert len(out.token_ids) == 10
    long_prompt = prompts_of(503, (30,), 9)[0]
    out = llm.generate(long_prompt, SamplingParams(temperature=0.0, max_new_tokens=1, ignore_eos=True))
    assert out.prompt_token_ids == long_prompt[-16:]
    # stream yields one record per token, the last one finished with its counts
    recs = list(llm.stream(prompt, SamplingParams(temperature=0.0, max_new_tokens=4, ignore_eos=True)))
    assert [r.token_id for r in recs] == greedy[:4] and [r.is_finished for r in recs] == [False] * 3 + [True]
    assert recs[-1].num_prompt_tokens == 6 and recs[-1].num_generated_tokens == 4
    # abort frees everything
    eng = llm.engine
    eng.add_request("gone", prompt, SamplingParams(max_new_tokens=50))
    eng.step()
    llm.abort("gone")
    assert not eng.has_unfinished_requests() and eng.runner.cache.num_free_pages() == 64
    with pytest.raises(ValueError):
        eng.add_request("bad", [503], SamplingParams())


def test_scheduling_ahead_changes_no_token(model_dirs, plain_models):
    """The next step is scheduled and packed while the device still samples the current one; with
    stop tokens that end requests unannounced, so few pages that requests are preempted, and an
    abort in between, every request gets the tokens and the ending it gets without that overlap."""
    from ullm_amd import FinishReason, SamplingParams
    cfg, w = plain_models["B"]
    prompts = prompts_of(503, (20, 3, 18, 9, 1, 14), 21)
    greedy = [plain.greedy_generate(w, cfg, p, 14) for p in prompts]
    # requests 0 and 3 stop on a token of their own continuation, 1 by max_tokens, the rest by max_new_tokens
    params = [SamplingParams(temperature=0.0, max_new_tokens=14, eos_token_id=greedy[0][5]),
              SamplingParams(temperature=0.0, max_tokens=9, ignore_eos=True),
              SamplingParams(temperature=0.0, max_new_tokens=14, ignore_eos=True),
              SamplingParams(temperature=0.0, max_new_tokens=14, eos_token_id=greedy[3][0]),
              SamplingParams(temperature=0.0, max_new_tokens=14, ignore_eos=True),
              SamplingParams(temperature=0.7, max_new_tokens=14, ignore_eos=True, seed=5)]
    runs = {}
    for ahead in (False, True):
        llm = make_llm(model_dirs["B"], page_size=4, num_pages=12, max_num_batched_tokens=16, max_prefill_chunk=7,
                       disable_async_scheduling=not ahead)
        eng = llm.engine
        for i, (p, sp) in enumerate(zip(prompts, params)):
            eng.add_request(f"r{i}", p, sp)
        got, steps = {}, 0
        while eng.has_unfinished_requests():
            for r in eng.step():
                rec = got.setdefault(r.seq_id, [[], None])
                if r.new_token_id >= 0:
                    rec[0].append(r.new_token_id)
                if r.is_finished:
                    rec[1] = r.finish_reason
            steps += 1
            if steps == 6:
                eng.abort_request("r4")
        assert eng.runner.cache.num_free_pages() == 12
        eng.runner.cache.check()
        runs[ahead] = (got, eng.scheduler.num_preemptions)
    plain_run, ahead_run = runs[False][0], runs[True][0]
    aborted = {k: v for k, v in ahead_run.items() if k == "r4"}
    for k in ("r0", "r1", "r2", "r3", "r5"):
        assert ahead_run[k] == plain_run[k], k
    assert ahead_run["r0"][0] == greedy[0][:greedy[0].index(greedy[0][5]) + 1] and ahead_run["r0"][1] is FinishReason.STOP
    assert ahead_run["r3"][0] == greedy[3][:1] and ahead_run["r3"][1] is FinishReason.STOP
    assert ahead_run["r1"][0] == greedy[1][:6] and ahead_run["r1"][1] is FinishReason.LENGTH
    assert ahead_run["r2"][0] == greedy[2] and ahead_run["r2"][1] is FinishReason.LENGTH
    assert all(v[1] is None for v in aborted.values())            # an aborted request reports no ending
    assert runs[True][1] > 0 and runs[False][1] > 0               # both runs had to preempt


@pytest.mark.parametrize("pages", [9, 11, 13])
def test_stop_tokens_while_requests_are_preempted(model_dirs, plain_models, pages):
    """Every request stops on a token of its own continuation while pages are so scarce that the
    youngest requests are preempted again and again (also in the very step that samples their stop
    token, and while the step after it is already queued): each ends where the plain continuation
    first shows its stop token, with and without the overlap, and all pages come back."""
    from ullm_amd import FinishReason, SamplingParams
    cfg, w = plain_models["B"]
    prompts = prompts_of(503, (13, 6, 9, 3, 11, 5, 8), 33)
    greedy = [plain.greedy_generate(w, cfg, p, 12) for p in prompts]
    stops = [g[k] for g, k in zip(greedy, (9, 3, 6, 11, 4, 8, 2))]
    want = [g[:g.index(t) + 1] for g, t in zip(greedy, stops)]
    preempted = 0
    for ahead in (False, True):
        llm = make_llm(model_dirs["B"], page_size=4, num_pages=pages, max_num_batched_tokens=12, max_prefill_chunk=5,
                       disable_async_scheduling=not ahead)
        eng = llm.engine
        for i, (p, t) in enumerate(zip(prompts, stops)):
            eng.add_request(f"r{i}", p, SamplingParams(temperature=0.0, max_new_tokens=12, eos_token_id=t))
        got, steps = {}, 0
        while eng.has_unfinished_requests():
            for r in eng.step():
                rec = got.setdefault(r.seq_id, [[], None])
                if r.new_token_id >= 0:
                    rec[0].append(r.new_token_id)
                if r.is_finished:
                    rec[1] = r.finish_reason
            steps += 1
            assert steps < 3000
        for i in range(len(prompts)):
            assert got[f"r{i}"] == [want[i], FinishReason.STOP], (ahead, i)
        assert eng.runner.cache.num_free_pages() == pages
        eng.runner.cache.check()
        preempted += eng.scheduler.num_preemptions
    assert preempted > 0


@pytest.mark.parametrize("ahead", [False, True])
def test_a_request_preempted_while_its_stop_token_is_sampled_ends_there(model_dirs, plain_models, ahead):
    """Three requests need a new page in the same step and none is free: the youngest loses its pages to
    the two older ones, in the planning round in which its third token, its stop token as it turns
    out, is still on the device.  When the token arrives the request ends; it is not run again."""
    from ullm_amd import FinishReason, SamplingParams
    cfg, w = plain_models["B"]
    for seed in range(40, 60):                       # a youngest request whose third token is new to its continuation
        prompts = prompts_of(503, (14, 14, 6), seed)
        third = plain.greedy_generate(w, cfg, prompts[2], 3)
        if third[2] not in third[:2]:
            break
    greedy = [plain.greedy_generate(w, cfg, p, 6) for p in prompts[:2]]
    llm = make_llm(model_dirs["B"], page_size=4, num_pages=10, max_num_batched_tokens=64, max_prefill_chunk=64,
                   disable_async_scheduling=not ahead)
    eng = llm.engine
    for i in range(2):
        eng.add_request(f"r{i}", prompts[i], SamplingParams(temperature=0.0, max_new_tokens=6, ignore_eos=True))
    eng.add_request("r2", prompts[2], SamplingParams(temperature=0.0, max_new_tokens=10, eos_token_id=third[2]))
    got, steps = {}, 0
    while eng.has_unfinished_requests():
        for r in eng.step():
            rec = got.setdefault(r.seq_id, [[], None])
            if r.new_token_id >= 0:
                rec[0].append(r.new_token_id)
            if r.is_finished:
                rec[1] = r.finish_reason
        steps += 1
        assert steps < 200
    assert eng.scheduler.num_preemptions == (1 if ahead else 0)     # in turn, the stop token is known before the pages run out
    assert got["r2"] == [third, FinishReason.STOP]
    assert got["r0"] == [greedy[0], FinishReason.LENGTH] and got["r1"] == [greedy[1], FinishReason.LENGTH]
    assert eng.runner.cache.num_free_pages() == 10
    eng.runner.cache.check()


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_scheduling_ahead_under_random_arrivals_and_aborts(model_dirs, seed):
    """Requests arrive while others run, some are aborted, pages are scarce and prefixes are shared:
    with and without the overlap every request that was not aborted gets the same tokens and the
    same ending, and all pages come back."""
    import random
    from ullm_amd import SamplingParams
    rng = random.Random(seed)
    n = 14
    common = [rng.randrange(503) for _ in range(9)]
    prompts = [(common if rng.random() < 0.4 else []) + [rng.randrange(503) for _ in range(rng.randint(1, 30))]
               for _ in range(n)]
    params = [SamplingParams(temperature=rng.choice([0.0, 0.8]), top_k=rng.choice([-1, 20]), seed=50 + i,
                             max_new_tokens=rng.randint(1, 12), eos_token_id=rng.randrange(503),
                             ignore_eos=rng.random() < 0.5) for i in range(n)]
    arrive = sorted(rng.randint(0, 25) for _ in range(n))              # step at which each request is added
    aborts = {rng.randrange(n): rng.randint(3, 30) for _ in range(3)}   # request -> step of its abort
    runs = []
    for ahead in (False, True):
        llm = make_llm(model_dirs["B"], page_size=4, num_pages=40, max_num_batched_tokens=20, max_prefill_chunk=9,
                       max_bs=5, enable_prefix_cache=True, disable_async_scheduling=not ahead)
        eng = llm.engine
        got, step, added = {}, 0, 0
        while added < n or eng.has_unfinished_requests():
            while added < n and arrive[added] <= step:
                eng.add_request(f"r{added}", prompts[added], params[added])
                added += 1
            for i, when in aborts.items():
                if when == step:
                    eng.abort_request(f"r{i}")
            for r in eng.step():
                rec = got.setdefault(r.seq_id, [[], None])
                if r.new_token_id >= 0:
                    rec[0].append(r.new_token_id)
                if r.is_finished:
                    rec[1] = r.finish_reason
            step += 1
            assert step < 2000
        eng.runner.cache.check()
        runs.append(got)
    plain_run, ahead_run = runs
    kept = [f"r{i}" for i in range(n) if i not in aborts]
    for k in kept:
        assert ahead_run[k] == plain_run[k] and ahead_run[k][1] is not None, k


def untied(tmp_path, name, seed):
    """The tiny configuration with an output matrix of its own (a tied one mostly predicts the token it was
    given, so greedy continuations would repeat one token and every stop token would come first)."""
    from conftest import CONFIGS
    from ullm_amd.weights.random_init import write_random_model
    d = write_random_model(dict(CONFIGS[name][0], tie_word_embeddings=False), str(tmp_path / f"untied{name}"), seed=seed)
    return d, plain.load_model_folder(d)


def run_and_check_own_path(llm, cfg, w, prompts, params, abort=None, rel=3e-2):
    """Run the requests to the end and check every request along the path it took itself: the logits the
    engine sampled from are the plain implementation's for the request's own tokens so far, every greedy token
    is the first largest of those logits, and the request ended where its rules say.  (In bfloat16 a near-tie
    may go the other way than in 32-bit, so tokens are not compared with a 32-bit run.)"""
    from ullm_amd import FinishReason
    eng = llm.engine
    seen = {}

    def hook(sampling, logits):
        for s_, row in zip(sampling, logits.float().cpu()):
            seen.setdefault(s_.request.request_id, []).append((s_.request.num_tokens, row))
    eng.on_logits = hook
    for i, (p, sp) in enumerate(zip(prompts, params)):
        eng.add_request(f"r{i}", p, sp)
    got, steps = {}, 0
    while eng.has_unfinished_requests():
        for r in eng.step():
            rec = got.setdefault(r.seq_id, [[], None])
            if r.new_token_id >= 0:
                rec[0].append(r.new_token_id)
            if r.is_finished:
                rec[1] = r.finish_reason
        steps += 1
        if abort is not None and steps == abort[1]:
            eng.abort_request(abort[0])
        assert steps < 3000
    checked = 0
    for i, (p, sp) in enumerate(zip(prompts, params)):
        rid = f"r{i}"
        tokens, reason = got.get(rid, [[], None])
        if abort is not None and rid == abort[0]:
            assert reason is None
            continue
        seq = p + tokens
        full = plain.qwen3_forward(w, cfg, seq)
        bound = rel * float(full.abs().max()) + 1e-6
        for pos, row in seen[rid]:
            if pos >= len(seq):
                continue                     # a token computed for a request that had already met its stop token
            assert float((row - full[pos - 1]).abs().max()) <= bound, (rid, pos)
            assert seq[pos] == int(row.argmax()), (rid, pos)
            checked += 1
        assert len(tokens) >= 1
        stops = {sp.eos_token_id} | set(sp.stop_token_ids) if not sp.ignore_eos else set()
        hit = [k for k, t_ in enumerate(tokens) if t_ in stops]
        if hit:
            assert hit[0] == len(tokens) - 1 and reason is FinishReason.STOP, (rid, tokens)
        else:
            assert reason is FinishReason.LENGTH, rid
            limits = [sp.max_new_tokens or 10 ** 9, (sp.max_tokens or 10 ** 9) - len(p)]
            assert len(tokens) == min(limits), (rid, tokens)
    return got, checked


@pytest.mark.parametrize("name,pages", [("D", 8), ("D", 9), ("E", 5)])
def test_bfloat16_generation_under_preemption_with_stop_tokens(tmp_path, name, pages):
    """The bfloat16 product path as generation runs it: matrix-core attention (head sizes 64 and 128, pages
    of 16, in E with a window whose pages are given back), decode steps replayed from graphs, token ids fed
    from the sampler's output on the device, so few pages that the youngest requests are preempted and
    recomputed, and stop tokens that end requests unannounced; with and without steps queued ahead."""
    from ullm_amd import SamplingParams
    d, (cfg, w) = untied(tmp_path, name, 21)
    prompts = prompts_of(cfg["vocab_size"], (13, 14, 15, 12, 11, 15, 14), 33)        # all but one cross a page's edge
    greedy = [plain.greedy_generate(w, cfg, p, 12) for p in prompts]
    # each request's stop token: the last token of its 32-bit continuation that had not occurred before
    stops = [g[max(k for k in range(12) if g.index(g[k]) == k)] for g in greedy]
    preempted = graphs = stopped = 0
    for ahead in (False, True):
        # a budget that admits all seven at once (a page each), portions of five: they then grow together
        llm = make_llm(d, dtype="bfloat16", page_size=16, num_pages=pages, max_num_batched_tokens=128,
                       max_prefill_chunk=5, disable_async_scheduling=not ahead)
        params = [SamplingParams(temperature=0.0, max_new_tokens=12, eos_token_id=t) for t in stops]
        got, checked = run_and_check_own_path(llm, cfg, w, prompts, params)
        eng = llm.engine
        assert checked >= 20
        stopped += sum(1 for v in got.values() if v[1].name == "STOP")
        for g in range(len(eng.runner.cache.groups)):
            assert eng.runner.cache.allocators[g].num_free == pages
        eng.runner.cache.check()
        preempted += eng.scheduler.num_preemptions
        graphs += len(eng.runner._graphs)
    assert preempted > 0
    assert graphs > 0
    assert stopped >= 4               # the bfloat16 runs met stop tokens too


def test_bfloat16_scheduling_ahead(tmp_path):
    """As the 32-bit test of scheduling ahead, on the bfloat16 path (config D with an output matrix of its
    own, pages of 16: matrix-core attention, graphs, ids fed on the device): stop tokens, length limits,
    scarce pages, an abort in between."""
    from ullm_amd import SamplingParams
    d, (cfg, w) = untied(tmp_path, "D", 22)
    prompts = prompts_of(cfg["vocab_size"], (20, 3, 18, 9, 1, 14), 21)
    greedy = [plain.greedy_generate(w, cfg, p, 14) for p in prompts]
    preempted = 0
    for ahead in (False, True):
        params = [SamplingParams(temperature=0.0, max_new_tokens=14, eos_token_id=greedy[0][5]),
                  SamplingParams(temperature=0.0, max_tokens=9, ignore_eos=True),
                  SamplingParams(temperature=0.0, max_new_tokens=14, ignore_eos=True),
                  SamplingParams(temperature=0.0, max_new_tokens=14, eos_token_id=greedy[3][0]),
                  SamplingParams(temperature=0.0, max_new_tokens=14, ignore_eos=True),
                  SamplingParams(temperature=0.0, max_new_tokens=14, ignore_eos=True)]
        llm = make_llm(d, dtype="bfloat16", page_size=16, num_pages=7, max_num_batched_tokens=64,
                       max_prefill_chunk=7, disable_async_scheduling=not ahead)
        got, checked = run_and_check_own_path(llm, cfg, w, prompts, params, abort=("r4", 6))
        assert checked >= 30
        assert llm.engine.runner.cache.num_free_pages() == 7
        llm.engine.runner.cache.check()
        preempted += llm.engine.scheduler.num_preemptions
    assert preempted > 0


def test_profile_start_stop_writes_a_trace(model_dirs, tmp_path):
    from ullm_amd import SamplingParams
    if DEV == "cpu":
        pytest.skip("the profiler records device activity")
    llm = make_llm(model_dirs["A"], profile=True, profile_dir=str(tmp_path / "traces"))
    llm.profile("start")
    llm.generate([[1, 2, 3]], SamplingParams(temperature=0.0, max_new_tokens=3, ignore_eos=True))
    llm.profile("stop")
    llm.profile("stop")                                  # a second stop is ignored
    assert any(f.endswith(".json.gz") for f in os.listdir(tmp_path / "traces"))
    with pytest.raises(RuntimeError, match="profiling is off"):
        make_llm(model_dirs["A"]).profile("start")


def test_prefix_cache_gives_the_same_tokens(model_dirs, plain_models):
    from ullm_amd import SamplingParams
    cfg, w = plain_models["A"]
    shared = prompts_of(256, (40,), 10)[0]
    prompts = [shared + [1, 2, 3], shared + [9], shared[:33]]
    llm = make_llm(model_dirs["A"], enable_prefix_cache=True, num_pages=32)
    sp = SamplingParams(temperature=0.0, max_new_tokens=5, ignore_eos=True)
    first = llm.generate(prompts[0], sp)
    rest = llm.generate(prompts[1:], sp)
    for p, o in zip(prompts, [first] + rest):
        assert o.token_ids == plain.greedy_generate(w, cfg, p, 5)
    assert llm.engine.runner.cache.prefix_tree.num_nodes >= 2
    llm.engine.runner.cache.check()


def test_bfloat16_prefix_cache_along_each_requests_own_path(tmp_path):
    """Prefix sharing on the bfloat16 path (config D, head size 64, pages of 16): a first portion that starts
    behind shared pages goes through the matrix-core prompt kernel with keys it did not write itself.  Requests
    share 40, 40 and 33 tokens of a prompt (two whole pages), one shares nothing; each is checked along its own
    path against the plain implementation, and the shared pages must have been found, not recomputed."""
    from ullm_amd import SamplingParams
    d, (cfg, w) = untied(tmp_path, "D", 23)
    shared = prompts_of(cfg["vocab_size"], (40,), 10)[0]
    other = prompts_of(cfg["vocab_size"], (21,), 11)[0]
    llm = make_llm(d, dtype="bfloat16", page_size=16, num_pages=32, enable_prefix_cache=True, max_prefill_chunk=24)
    sp = SamplingParams(temperature=0.0, max_new_tokens=6, ignore_eos=True)
    _, checked = run_and_check_own_path(llm, cfg, w, [shared + [1, 2, 3]], [sp])
    tree = llm.engine.runner.cache.prefix_tree
    assert tree.num_nodes >= 2
    eng = llm.engine
    computed = []
    launch = eng.runner.launch

    def counting(prepared):
        computed.append(sum(len(e.tokens) for e in prepared.entries))
        return launch(prepared)
    eng.runner.launch = counting
    prompts = [shared + [9], shared[:33] + [7, 7], other, shared + [1, 2, 3, 4]]
    for i, p in enumerate(prompts):                      # under fresh ids: the checker names requests r0, r1, ...
        eng.add_request(f"r{i}", p, sp)
    got = {}
    seen = {}
    eng.on_logits = lambda sampling, logits: [seen.setdefault(s_.request.request_id, []).append((s_.request.num_tokens, row))
                                              for s_, row in zip(sampling, logits.float().cpu())]
    while eng.has_unfinished_requests():
        for r in eng.step():
            if r.new_token_id >= 0:
                got.setdefault(r.seq_id, []).append(r.new_token_id)
    for i, p in enumerate(prompts):
        seq = p + got[f"r{i}"]
        full = plain.qwen3_forward(w, cfg, seq)
        bound = 3e-2 * float(full.abs().max()) + 1e-6
        for pos, row in seen[f"r{i}"]:
            if pos >= len(seq):
                continue
            assert float((row - full[pos - 1]).abs().max()) <= bound, (i, pos)
            assert seq[pos] == int(row.argmax()), (i, pos)
            checked += 1
    assert checked >= 30
    # 41 + 35 + 21 + 44 prompt tokens and 4 x 5 decoded ones; two pages of 16 were found for three of the requests
    assert sum(computed) == 41 + 35 + 21 + 44 + 4 * 5 - 3 * 32, computed
    eng.runner.cache.check()


def test_command_line(model_dirs, plain_models, capsys):
    from ullm_amd.cli import main
    cfg, w = plain_models["A"]
    rc = main(["--model", model_dirs["A"], "--dtype", "float32", "--prompt-ids", "5,17,3", "--prompt-ids", "9,8",
               "--temperature", "0", "--max-new-tokens", "4", "--ignore-eos", "--context-len", "64", "--num-pages", "16",
               "--max-bs", "4"])
    assert rc == 0
    lines = [json.loads(x) for x in capsys.readouterr().out.strip().splitlines() if x.startswith("{")]
    assert [x["token_ids"] for x in lines] == [plain.greedy_generate(w, cfg, [5, 17, 3], 4),
                                               plain.greedy_generate(w, cfg, [9, 8], 4)]


def test_command_line_with_random_weights(tmp_path, capsys):
    """``--random-weights CONFIG.JSON:SEED`` draws the weights on the device: the same seed gives the same tokens,
    another seed other tokens."""
    from conftest import TINY_B
    from ullm_amd.cli import main
    path = tmp_path / "config.json"
    path.write_text(json.dumps(TINY_B))
    runs = []
    for seed in (4, 4, 5):
        rc = main(["--random-weights", f"{path}:{seed}", "--dtype", "float32", "--prompt-ids", "5,17,3,99,200",
                   "--temperature", "0", "--max-new-tokens", "6", "--ignore-eos", "--context-len", "64", "--num-pages", "16",
                   "--max-bs", "4"])
        assert rc == 0
        lines = [json.loads(x) for x in capsys.readouterr().out.strip().splitlines() if x.startswith("{")]
        runs.append(lines[0]["token_ids"])
    assert len(runs[0]) == 6 and runs[0] == runs[1] and runs[0] != runs[2]


@pytest.mark.parametrize("trial", range(10))
def test_random_engine_settings_change_no_token(tmp_path, trial):
    """The same requests (seeded sampling, stop ids, every kind of length limit) through a roomy engine that runs
    eagerly and waits for every step, and through one with settings drawn at random (pages for little more than
    one request, small budgets and portions, prefix sharing, graphs, steps queued ahead); requests join while
    others run and one may be aborted.  In 32-bit: the same tokens and the same reasons to stop."""
    import random
    from ullm_amd import LLM, EngineConfig, SamplingParams
    from ullm_amd.weights.random_init import write_random_model
    rng = random.Random(77000 + trial)
    nkv = rng.choice([1, 2, 4])
    cfg = dict(architectures=["Qwen3ForCausalLM"], hidden_size=rng.choice([40, 72, 96]), num_hidden_layers=rng.choice([1, 2]),
               num_attention_heads=nkv * rng.choice([1, 2, 4]), num_key_value_heads=nkv, head_dim=rng.choice([16, 32, 64, 128]),
               intermediate_size=rng.choice([56, 104]), vocab_size=rng.choice([31, 101, 257]), rope_theta=1e4,
               rms_norm_eps=1e-6, max_position_embeddings=512, tie_word_embeddings=rng.random() < 0.5,
               initializer_range=0.08, use_sliding_window=rng.random() < 0.3, sliding_window=rng.choice([7, 33]),
               max_window_layers=rng.choice([0, 1]))
    stop_ids = rng.choice([None, 3, [3, 5, 9]])
    if stop_ids is not None:
        cfg["eos_token_id"] = stop_ids
    d = write_random_model(cfg, str(tmp_path / "m"), seed=trial)
    V, page_size, n_req = cfg["vocab_size"], rng.choice([4, 8, 16]), rng.choice([2, 5, 9, 14])
    shared = [rng.randrange(V) for _ in range(rng.choice([0, 0, 9, 40]))]
    prompts = [shared + [rng.randrange(V) for _ in range(rng.choice([1, 2, 5, 17, 40, 70]))] for _ in range(n_req)]
    params = []
    for p in prompts:
        kw = dict(temperature=rng.choice([0.0, 0.7, 1.0, 1.5]), top_k=rng.choice([-1, 5, 20]), top_p=rng.choice([1.0, 0.9]),
                  min_p=rng.choice([0.0, 0.05]), seed=rng.randrange(1 << 20), ignore_eos=rng.random() < 0.3,
                  stop_token_ids=rng.choice([[], [], [1, 2], [rng.randrange(V)]]))
        limit = rng.choice(["new", "total", "both", "context"])
        if limit in ("new", "both"):
            kw["max_new_tokens"] = rng.choice([1, 2, 8, 30, 60])
        if limit in ("total", "both"):
            kw["max_tokens"] = len(p) + rng.choice([1, 3, 25])
        if rng.random() < 0.3:
            kw["eos_token_id"] = rng.randrange(V)
        params.append(SamplingParams(**kw))
    context_len = 160
    one_request = -(-context_len // page_size) + 1
    pages = rng.choice([one_request, one_request + 3, 2 * one_request, 8 * one_request])
    base = dict(model=d, dtype="float32", context_len=context_len, page_size=page_size, device=DEV)
    ids = [f"q{i}" for i in range(n_req)]
    roomy = LLM(EngineConfig(**base, max_bs=16, num_pages=16 * one_request, enforce_eager=True, disable_async_scheduling=True))
    want = roomy.generate(prompts, params, ids)
    eng = LLM(EngineConfig(**base, max_bs=rng.choice([2, 4, 8, 16]), num_pages=pages,
                           max_num_batched_tokens=rng.choice([8, 16, 33, 256]), max_prefill_chunk=rng.choice([3, 7, 16, 256]),
                           enable_prefix_cache=rng.random() < 0.5, enforce_eager=rng.random() < 0.4,
                           disable_async_scheduling=rng.random() < 0.3)).engine
    abort = rng.randrange(n_req) if rng.random() < 0.3 and n_req > 2 else None
    got, pending, steps = {}, list(range(n_req)), 0
    while pending or eng.has_unfinished_requests():
        for _ in range(rng.choice([0, 1, 1, 3])):
            if pending:
                i = pending.pop(0)
                eng.add_request(ids[i], prompts[i], params[i])
        if not eng.has_unfinished_requests():
            continue
        for out in eng.step():
            got.setdefault(out.seq_id, []).append(out)
        steps += 1
        assert steps < 5000
        if abort is not None and steps == 3:
            if ids[abort] in eng.scheduler.requests:
                eng.abort_request(ids[abort])
            else:
                abort = None
    for i in range(n_req):
        if i == abort:
            continue
        assert [o.new_token_id for o in got[ids[i]]] == want[i].token_ids
        assert got[ids[i]][-1].finish_reason == want[i].finish_reason
    eng.runner.cache.check()
    assert eng.config.enable_prefix_cache or eng.runner.cache.num_free_pages() == pages

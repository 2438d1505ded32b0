"""The scheduler's decisions, driven without a model: a fake step appends token 1 to every request
whose share reaches its end (no GPU)."""
import pytest

from ullm_amd.cache.manager import CacheGroupSpec, CacheManager
from ullm_amd.engine.request import FinishReason, Request, RequestStatus
from ullm_amd.engine.scheduler import Scheduler
from ullm_amd.sampling import SamplingParams


def make(num_pages=64, page_size=4, max_bs=4, budget=16, chunk=8, prefix=False):
    cache = CacheManager([CacheGroupSpec(2, 16, 0, (0,))], [num_pages], page_size, max_bs, enable_prefix_cache=prefix)
    return Scheduler(cache, budget, chunk, max_bs), cache


def req(i, n_prompt, **kw):
    return Request(f"r{i}", list(range(1, n_prompt + 1)), n_prompt, SamplingParams(**kw), seed=i, order=i)


def run_step(sched, cache, max_new=None, log=None):
    """schedule, pretend to run, append a token where the share reached the end."""
    out = sched.schedule()
    if log is not None:
        log.append([(s.request.request_id, s.start, s.num_tokens) for s in out])
    for s in out:
        cache.commit(s.request.cache, s.num_tokens)
    for s in out:
        if s.samples:
            sched.append_token(s.request, 1)
            if max_new is not None and s.request.num_generated_tokens >= max_new:
                sched.finish(s.request)
    cache.check()
    return out


def test_prompts_are_cut_under_the_budget_and_chunk():
    sched, cache = make(budget=16, chunk=8)
    sched.add(req(0, 21))
    log = []
    run_step(sched, cache, log=log)
    run_step(sched, cache, log=log)
    run_step(sched, cache, log=log)
    run_step(sched, cache, log=log)
    assert log == [[("r0", 0, 8)], [("r0", 8, 8)], [("r0", 16, 5)], [("r0", 21, 1)]]


def test_fcfs_and_budget_shared_between_decodes_and_portions():
    sched, cache = make(budget=10, chunk=8)
    for i, n in enumerate([3, 12, 4]):
        sched.add(req(i, n))
    log = []
    run_step(sched, cache, log=log)
    # r0 whole (3), r1 gets the rest of the budget (7), r2 must wait: no overtaking
    assert log[0] == [("r0", 0, 3), ("r1", 0, 7)]
    run_step(sched, cache, log=log)
    # r0 decodes first (1 token), then r1's portion (5 left of 12), then r2 is admitted with what is left
    assert log[1] == [("r0", 3, 1), ("r1", 7, 5), ("r2", 0, 4)]
    run_step(sched, cache, log=log)
    assert log[2] == [("r0", 4, 1), ("r1", 12, 1), ("r2", 4, 1)]
    for step in log:
        assert sum(n for _, _, n in step) <= 10
        assert len({r for r, _, _ in step}) == len(step)          # each request at most once per step


def test_decodes_never_starve_behind_a_long_prompt():
    sched, cache = make(num_pages=200, budget=8, chunk=8)
    sched.add(req(0, 2))
    run_step(sched, cache)
    sched.add(req(1, 100))
    for _ in range(10):
        out = run_step(sched, cache)
        assert out[0].request.request_id == "r0" and out[0].num_tokens == 1
        assert out[1].request.request_id == "r1" and out[1].num_tokens == 7


def test_max_bs_bounds_the_running_set():
    sched, cache = make(max_bs=2, budget=100, chunk=100)
    for i in range(4):
        sched.add(req(i, 3))
    out = run_step(sched, cache, max_new=2)
    assert [s.request.request_id for s in out] == ["r0", "r1"]
    run_step(sched, cache, max_new=2)              # both finish here
    out = run_step(sched, cache, max_new=2)
    assert [s.request.request_id for s in out] == ["r2", "r3"]


def test_one_token_prompt_works():
    sched, cache = make(prefix=True)
    sched.add(req(0, 1))
    out = run_step(sched, cache)
    assert [(s.start, s.num_tokens, s.samples) for s in out] == [(0, 1, True)]


def test_pages_run_out_the_youngest_is_preempted_and_recomputed():
    # 6 pages of 4 tokens: two requests of 8 tokens fill 4 pages, both decode until the pool is full
    sched, cache = make(num_pages=6, page_size=4, budget=32, chunk=32)
    sched.add(req(0, 8))
    sched.add(req(1, 8))
    log = []
    for _ in range(12):
        run_step(sched, cache, log=log)
    r0, r1 = sched.requests["r0"], sched.requests["r1"]
    assert r1.num_preemptions >= 1 and r0.num_preemptions == 0
    # after its preemption r1 waits at the front and holds nothing
    pre = next(i for i, step in enumerate(log) if all(r != "r1" for r, _, _ in step))
    assert pre > 0
    # r0 went on decoding without a gap
    assert all(any(r == "r0" for r, _, _ in step) for step in log)
    # when r1 comes back it is recomputed from all its tokens, prompt and generated
    back = next((step for step in log[pre:] if any(r == "r1" for r, _, _ in step)), None)
    if back is not None:
        start, n = next((s, n) for r, s, n in back if r == "r1")
        assert start == 0 and n > 8
    cache.check()


def test_a_request_alone_that_cannot_grow_ends_with_length():
    sched, cache = make(num_pages=2, page_size=4, budget=32, chunk=32)
    sched.add(req(0, 6))
    for _ in range(10):
        run_step(sched, cache)
        if not sched.has_unfinished():
            break
    assert not sched.has_unfinished()
    done = sched.finished_by_scheduler[0]
    assert done.finish_reason is FinishReason.LENGTH and done.num_tokens == 9    # 8 cached + 1 it could not place
    assert cache.num_free_pages() == 2


def test_a_prompt_larger_than_the_pool_is_refused_at_once():
    sched, cache = make(num_pages=2, page_size=4)
    with pytest.raises(ValueError, match="needs 3 pages"):
        sched.add(req(0, 9))
    with pytest.raises(ValueError, match="already in use"):
        sched.add(req(1, 2)) or sched.add(req(1, 2))


def test_admission_stops_when_pages_are_short_without_preempting():
    sched, cache = make(num_pages=4, page_size=4, budget=64, chunk=64)
    sched.add(req(0, 10))                                  # 3 pages
    sched.add(req(1, 7))                                   # needs 2, only 1 left
    out = run_step(sched, cache)
    assert [s.request.request_id for s in out] == ["r0"]
    assert sched.requests["r1"].status is RequestStatus.WAITING and sched.requests["r0"].num_preemptions == 0
    assert cache.num_free_slots == 3                       # the slot tried for r1 was given back


def test_abort_from_any_state():
    sched, cache = make()
    sched.add(req(0, 5))
    sched.add(req(1, 5))
    run_step(sched, cache)
    sched.add(req(2, 5))
    sched.finish(sched.requests["r0"])                     # running
    sched.finish(sched.requests["r2"])                     # waiting
    assert [r.request_id for r in sched.running] == ["r1"] and not sched.waiting
    cache.check()


def test_prefix_sharing_skips_cached_pages_at_admission():
    sched, cache = make(prefix=True, budget=64, chunk=64)
    sched.add(req(0, 10))
    run_step(sched, cache, max_new=1)                      # finishes, its 2 full pages go to the tree
    sched.add(req(1, 10))                                  # the same tokens
    out = run_step(sched, cache)
    assert [(s.start, s.num_tokens) for s in out] == [(8, 2)]


def test_batch_buckets_of_the_captured_decode_graphs():
    """A decode step replays the graph of the next bucket: never smaller than the batch, less than half as large again
    from 33 requests on, and the same bucket for every batch up to it."""
    from ullm_amd.engine.runner import batch_bucket
    assert [batch_bucket(n) for n in (1, 2, 3, 8, 9, 16, 17, 32)] == [1, 2, 4, 8, 16, 16, 32, 32]
    assert [batch_bucket(n) for n in (33, 48, 49, 64, 65, 96, 97, 128, 129, 192, 193, 256)] == \
        [48, 48, 64, 64, 96, 96, 128, 128, 192, 192, 256, 256]
    for n in range(1, 600):
        b = batch_bucket(n)
        assert b >= n and batch_bucket(b) == b and (n <= 32 or 2 * b < 3 * n)


def test_sampler_stages_one_word_for_the_host_beside_the_rows():
    """The staged parameters are seven words a row and one more that only the host reads: whether any row has
    settings that the sampling kernels serve by cutting rows into parts (all but greedy and a large top-k)."""
    import torch
    from ullm_amd.sampling import Sampler, SamplingParams
    sampler = Sampler(torch.device("cpu"))
    cases = [([SamplingParams(temperature=0.0)] * 3, False),
             ([SamplingParams(temperature=0.0), SamplingParams(temperature=0.7)], True),
             ([SamplingParams(temperature=0.7, top_p=0.9)], True),
             ([SamplingParams(temperature=0.7, top_p=0.9, min_p=0.1)], True),
             ([SamplingParams(temperature=0.7, top_k=20, top_p=0.9, min_p=0.05)], True),
             ([SamplingParams(temperature=0.7, top_k=100)], False),
             ([SamplingParams(temperature=0.7, min_p=0.1)], True)]
    for params, cut in cases:
        n = len(params)
        staged = sampler.stage(params, list(range(n)), [5] * n)
        assert staged.numel() == 7 * n + 1
        inputs = sampler.send(staged)
        assert inputs.n == n and inputs.packed.shape == (7, n) and inputs.cut_rows is cut
        assert inputs.packed[3].tolist() == [p.top_k for p in params]
        assert inputs.packed[6].tolist() == [5] * n

"""The engine at the layer widths it is tuned for (Qwen3-8B and Qwen3-32B: width 4096 / 5120, 32 / 64 query
heads over 8 kv heads of 128, vocabulary 151,936), two layers deep, with random weights bound in place.
Every choice of kernel by row count, matrix size, context length and batch bucket is keyed to these sizes,
so the tiny configurations never cross them: here bfloat16 (graphs and eager) is compared with the true
32-bit engine on the same weights, step by step, across prompt portions of many sizes and decode batches
on both sides of every row threshold."""
import pytest
import torch

from gpu_util import DEV

pytestmark = pytest.mark.gpu

SIZES = {
    "qwen3_8b": dict(hidden_size=4096, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
                     intermediate_size=12288),
    "qwen3_32b": dict(hidden_size=5120, num_attention_heads=64, num_key_value_heads=8, head_dim=128,
                      intermediate_size=25600),
}
LONG = 1100                 # tokens of the long contexts: past the 1,024 keys the attention kernels fetch page ids for at once
N_REQUESTS = 257


def _config(sizes):
    return dict(architectures=["Qwen3ForCausalLM"], num_hidden_layers=2, vocab_size=151936, rope_theta=1000000.0,
                rms_norm_eps=1e-6, max_position_embeddings=4096, tie_word_embeddings=False, attention_bias=False,
                use_sliding_window=False, initializer_range=0.02, torch_dtype="bfloat16", **sizes)


class Harness:
    """One runner over a model with random weights; requests are admitted on first use."""

    def __init__(self, config, dtype, use_graphs, share=None):
        from ullm_amd.engine.loading import make_env
        from ullm_amd.engine.runner import ModelRunner
        from ullm_amd.models import build_model
        from ullm_amd.weights.random_init import bind_random_weights
        if share is None:
            self.env = make_env(dtype, DEV, 2048)
            _, self.model = build_model(config)
            bind_random_weights(self.model, self.env, seed=0)
        else:
            self.env, self.model = share.env, share.model
        pages = (4 * 1280 + N_REQUESTS * 128) // 16
        self.runner = ModelRunner(self.model, self.env, page_size=16, num_pages=pages, max_requests=N_REQUESTS + 3,
                                  use_graphs=use_graphs)
        self.live = {}

    def step(self, entries):
        """entries: [(request id, tokens)]; returns the logits of every entry's last token (device)."""
        from ullm_amd.engine.runner import StepEntry
        batch = []
        for rid, tokens in entries:
            rc = self.live.get(rid)
            if rc is None:
                rc = self.live[rid] = self.runner.cache.admit(str(rid))
            assert self.runner.cache.reserve(rc, len(tokens))
            batch.append(StepEntry(rc, list(tokens), [len(tokens) - 1]))
        return self.runner.step(batch)


def _compare(got16, want32, what, rel=3e-2):
    """bfloat16 logits against 32-bit ones: within rel of the largest logit, and the same argmax on every
    row whose two largest 32-bit logits are further apart than twice that row's error."""
    assert torch.isfinite(got16).all() and torch.isfinite(want32).all(), what
    scale = float(want32.abs().max())
    err = (got16 - want32).abs().amax(dim=1)
    assert float(err.max()) <= rel * scale, f"{what}: max |diff| {float(err.max()):.4f} > {rel} * {scale:.3f}"
    top2 = want32.topk(2, dim=1).values
    clear = (top2[:, 0] - top2[:, 1]) > 2 * err
    same = got16.argmax(dim=1) == want32.argmax(dim=1)
    assert bool((same | ~clear).all()), f"{what}: argmax differs on rows {torch.nonzero(~same & clear).flatten().tolist()}"
    return int(clear.sum())


@pytest.mark.parametrize("size", sorted(SIZES))
def test_bfloat16_equals_the_32_bit_engine_at_real_widths(size):
    config = _config(SIZES[size])
    g = torch.Generator().manual_seed(1)
    lens = [LONG] * 4 + torch.randint(20, 61, (N_REQUESTS - 4,), generator=g).tolist()
    prompts = [torch.randint(0, config["vocab_size"], (n,), generator=g).tolist() for n in lens]
    tails = [torch.randint(0, config["vocab_size"], (12,), generator=g).tolist() for _ in lens]   # tokens to decode with
    graphs = Harness(config, "bfloat16", True)
    eager = Harness(config, "bfloat16", False, share=graphs)
    full = Harness(config, "float32", False)
    assert graphs.runner.use_graphs and not eager.runner.use_graphs
    # the same seed gave both dtypes the same weights
    assert torch.equal(graphs.model.blocks[1].ffn.w_gate_up.float(), full.model.blocks[1].ffn.w_gate_up)
    runners = (graphs, eager, full)

    def all_step(entries, what):
        a, b, c = (h.step(entries) for h in runners)
        decided = _compare(a, c, what + " (graphs)")
        _compare(b, c, what + " (eager)")
        _compare(a, b, what + " (graphs against eager)", rel=1.5e-2)
        return decided

    # prompts: whole (library products), and in portions on both sides of every row threshold of the projections
    decided = all_step([(0, prompts[0])], "a whole long prompt")
    done = {1: 0, 2: 0, 3: 0}
    portions = [8, 9, 16, 17, 32, 33, 64, 65, 256, 257, 2, 31]
    for i, n in enumerate(portions):
        rid = 1 + i % 3
        decided += all_step([(rid, prompts[rid][done[rid]:done[rid] + n])], f"a portion of {n} tokens")
        done[rid] += n
    rest = [(rid, prompts[rid][done[rid]:]) for rid in (1, 2, 3)]
    decided += all_step(rest, "three long portions in one step")
    for first in range(4, N_REQUESTS, 50):                       # the short prompts, fifty requests a step
        ids = range(first, min(first + 50, N_REQUESTS))
        decided += all_step([(r, prompts[r]) for r in ids], f"short prompts {first}..")
    # one token per request: batches on both sides of the thresholds (8 | 9 folded norm, 16 | 17 folded adds,
    # 32 | 33 gate|up, 64 | 65 and 256 | 257 the stacked products, 256 | 257 also the largest graph)
    used = [0] * N_REQUESTS
    for batch in (8, 9, 16, 17, 32, 33, 64, 65, 256, 257, 1, 128):
        entries = []
        for r in range(batch):
            entries.append((r, [tails[r][used[r]]]))
            used[r] += 1
        decided += all_step(entries, f"decode batch {batch}")
    assert len(graphs.runner._graphs) >= 6 and not eager.runner._graphs
    assert decided > 500          # most rows had a clear winner, so the argmax check was a real one
    for h in runners:
        h.runner.cache.check()

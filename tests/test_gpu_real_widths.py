"""The engine at the layer widths it is tuned for (Qwen3-8B, -14B and -32B: width 4096 / 5120, 32 / 40 / 64 query
heads over 8 kv heads of 128, vocabulary 151,936), one or two layers deep, with random weights.
Every choice of kernel by row count, matrix size, context length and batch bucket is keyed to these sizes,
so the tiny configurations never cross them: here bfloat16 (graphs and eager) is compared with the true
32-bit engine on the same weights, step by step, across prompt portions of many sizes and decode batches
on both sides of every row threshold; and one layer of each width, loaded from a folder, is compared in
32-bit and in bfloat16 with the plain implementation on the CPU, at every position."""
import pytest
import torch

from gpu_util import DEV

pytestmark = pytest.mark.gpu

SIZES = {
    "qwen3_8b": dict(hidden_size=4096, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
                     intermediate_size=12288),
    "qwen3_14b": dict(hidden_size=5120, num_attention_heads=40, num_key_value_heads=8, head_dim=128,
                      intermediate_size=17408),
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


CLEAR = 1e-2               # a row has a clear winner if its two largest 32-bit logits differ by more than 2 * CLEAR * largest |logit|


def _compare(got16, want32, what, rel=3e-2):
    """bfloat16 logits against 32-bit ones: within rel of the largest logit, and the same argmax on every row
    with a clear winner.  Which rows those are is decided by the 32-bit logits alone, not by the error found:
    a kernel that is further off has as many rows to answer for."""
    assert torch.isfinite(got16).all() and torch.isfinite(want32).all(), what
    scale = float(want32.abs().max())
    err = (got16 - want32).abs().amax(dim=1)
    assert float(err.max()) <= rel * scale, f"{what}: max |diff| {float(err.max()):.4f} > {rel} * {scale:.3f}"
    top2 = want32.topk(2, dim=1).values
    clear = (top2[:, 0] - top2[:, 1]) > 2 * CLEAR * scale
    same = got16.argmax(dim=1) == want32.argmax(dim=1)
    assert bool((same | ~clear).all()), f"{what}: argmax differs on rows {torch.nonzero(~same & clear).flatten().tolist()}"
    print(f"{what}: error {float(err.max()) / scale:.2e} of the largest logit, {int(clear.sum())} of {len(err)} rows clear")
    return int(clear.sum())


@pytest.mark.parametrize("size", sorted(SIZES))
def test_bfloat16_equals_the_32_bit_engine_at_real_widths(size):
    config = _config(SIZES[size])
    g = torch.Generator().manual_seed(1)
    lens = [LONG] * 4 + torch.randint(20, 61, (N_REQUESTS - 4,), generator=g).tolist()
    prompts = [torch.randint(0, config["vocab_size"], (n,), generator=g).tolist() for n in lens]
    tails = [torch.randint(0, config["vocab_size"], (14,), generator=g).tolist() for _ in lens]   # tokens to decode with
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
    for batch in (8, 9, 16, 17, 32, 33, 64, 65, 80, 96, 256, 257, 1, 128):
        entries = []
        for r in range(batch):
            entries.append((r, [tails[r][used[r]]]))
            used[r] += 1
        decided += all_step(entries, f"decode batch {batch}")
    assert len(graphs.runner._graphs) >= 6 and not eager.runner._graphs
    assert decided > 300          # rows with a clear winner: the argmax check had something to lose
    for h in runners:
        h.runner.cache.check()


def _write_folder(config, folder, seed):
    """A model folder for ``config`` written by this test alone: the checkpoint's own tensor names and
    shapes, drawn on the GPU in bfloat16 (matrices N(0, 0.02), gains 1 + N(0, 0.1)).  Returns the tensors
    widened to float32 on the CPU, for the plain implementation."""
    import json
    import os
    from safetensors.torch import save_file
    H, I, V = config["hidden_size"], config["intermediate_size"], config["vocab_size"]
    nq, nkv, hd = config["num_attention_heads"], config["num_key_value_heads"], config["head_dim"]
    shapes = {"model.embed_tokens.weight": (V, H), "lm_head.weight": (V, H), "model.norm.weight": (H,)}
    for layer in range(config["num_hidden_layers"]):
        p = f"model.layers.{layer}"
        shapes.update({f"{p}.input_layernorm.weight": (H,), f"{p}.post_attention_layernorm.weight": (H,),
                       f"{p}.self_attn.q_proj.weight": (nq * hd, H), f"{p}.self_attn.k_proj.weight": (nkv * hd, H),
                       f"{p}.self_attn.v_proj.weight": (nkv * hd, H), f"{p}.self_attn.o_proj.weight": (H, nq * hd),
                       f"{p}.self_attn.q_norm.weight": (hd,), f"{p}.self_attn.k_norm.weight": (hd,),
                       f"{p}.mlp.gate_proj.weight": (I, H), f"{p}.mlp.up_proj.weight": (I, H),
                       f"{p}.mlp.down_proj.weight": (H, I)})
    gen = torch.Generator(device=DEV).manual_seed(seed)
    stored = {}
    for name, shape in shapes.items():
        t = torch.empty(shape, dtype=torch.float32, device=DEV)
        if len(shape) == 1:
            t.normal_(0.0, 0.1, generator=gen).add_(1.0)
        else:
            t.normal_(0.0, 0.02, generator=gen)
        stored[name] = t.to(torch.bfloat16).cpu()
        del t
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(config, f)
    save_file(stored, os.path.join(folder, "model.safetensors"), metadata={"format": "pt"})
    return {k: v.float() for k, v in stored.items()}


@pytest.mark.parametrize("size", sorted(SIZES))
def test_one_layer_at_real_widths_equals_the_plain_implementation(size, tmp_path):
    """What the two precisions of the engine share (the loader's merging of q | k | v and gate | up, the packing of
    a batch, the rotary table, the embedding gather over 0.6 to 0.8 G elements, the 32-bit product at inner
    sizes up to 25,600) is outside a comparison of one with the other: here a folder with one layer of each
    width goes through the engine's own loader, 40 prompt tokens in portions of 17, 9 and 14 and then 6 single
    tokens through the step function, and the logits at all 46 positions are compared with the plain
    implementation's on the CPU."""
    import plain_qwen3 as plain
    from ullm_amd.engine.loading import load_model
    from ullm_amd.engine.runner import ModelRunner, StepEntry
    config = dict(_config(SIZES[size]), num_hidden_layers=1)
    weights = _write_folder(config, str(tmp_path), seed=3)
    g = torch.Generator().manual_seed(4)
    tokens = torch.randint(0, config["vocab_size"], (46,), generator=g).tolist()
    tokens[5], tokens[45] = 0, config["vocab_size"] - 1                      # the table's first and last row
    want = plain.qwen3_forward(weights, config, tokens)
    scale = float(want.abs().max())
    cuts = [17, 9, 14, 1, 1, 1, 1, 1, 1]
    for dtype, rel in (("float32", 2e-5), ("bfloat16", 3e-2)):
        _, model, env = load_model(str(tmp_path), dtype, DEV, 256)
        runner = ModelRunner(model, env, page_size=16, num_pages=8, max_requests=2, use_graphs=False)
        rc = runner.cache.admit("r")
        rows, at = [], 0
        for n in cuts:
            assert runner.cache.reserve(rc, n)
            rows.append(runner.step([StepEntry(rc, tokens[at:at + n], list(range(n)))]).cpu())
            at += n
        got = torch.cat(rows)
        assert got.shape == want.shape and torch.isfinite(got).all()
        err = (got - want).abs().amax(dim=1)
        worst = int(err.argmax())
        assert float(err.max()) <= rel * scale, \
            f"{size} {dtype}: position {worst} is {float(err.max()):.3e} from the plain logits, bound {rel * scale:.3e}"
        if dtype == "float32":
            assert torch.equal(got.argmax(dim=1), want.argmax(dim=1))
        runner.cache.release(rc)
        runner.cache.check()
        del runner, model
        torch.cuda.empty_cache()

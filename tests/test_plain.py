"""Pins of the plain implementation beside the reference's text: special cases that reduce to a
library routine, invariants, and the one worked example the reference holds.  Each is chosen so that
a plausible mistake (wrong sign or pairing, a norm in the wrong place, a wrong group mapping) fails.
The reference has no tests or vectors of its own (its only example is the prefix-tree comment,
checked in test_cache_manager.py), so the whole-model result is 'parity unpinned' against a run of
the reference: it is pinned through its parts."""
import math

import pytest
import torch
import torch.nn.functional as F

import plain_qwen3 as plain
from conftest import TINY_A, TINY_B, TINY_C


def test_rms_norm_is_the_library_routine():
    torch.manual_seed(0)
    x, w = torch.randn(5, 7, 48), torch.randn(48)
    for eps in (1e-6, 1e-3):
        assert torch.allclose(plain.rms_norm(x, w, eps), F.rms_norm(x, (48,), w, eps), atol=1e-6)
    # gain 1, eps 0: y = x * sqrt(n) / |x|
    y = plain.rms_norm(x, torch.ones(48), 0.0)
    assert torch.allclose(y, x * math.sqrt(48) / x.norm(dim=-1, keepdim=True), atol=1e-5)
    # scale invariance (fails if eps were added outside the root or the mean were a sum)
    assert torch.allclose(plain.rms_norm(7.0 * x, w, 0.0), plain.rms_norm(x, w, 0.0), atol=1e-5)


def test_rope_position_zero_is_identity_and_two_dims_is_a_plane_rotation():
    torch.manual_seed(1)
    x = torch.randn(1, 3, 16)
    cos, sin = plain.rope_cos_sin(torch.tensor([0]), 16, 10000.0)
    assert torch.allclose(plain.apply_rope_concat_layout(x, cos, sin), x)
    # head_dim 2: one pair, angle = p * base^0 = p: (a, b) -> (a cos p - b sin p, b cos p + a sin p)
    v = torch.tensor([[[1.0, 0.0]]])
    cos, sin = plain.rope_cos_sin(torch.tensor([3]), 2, 12345.0)
    out = plain.apply_rope_concat_layout(v, cos, sin)
    assert torch.allclose(out, torch.tensor([[[math.cos(3.0), math.sin(3.0)]]]), atol=1e-6)


def test_rope_angles_and_pairing():
    # angle of pair i at position p is p * theta^(-2i/d); pair i is (x[i], x[i + d/2])
    d, theta, p = 8, 100.0, 5
    cos, sin = plain.rope_cos_sin(torch.tensor([p]), d, theta)
    for i in range(d // 2):
        ang = p * theta ** (-2.0 * i / d)
        assert abs(cos[0, i].item() - math.cos(ang)) < 1e-5 and abs(sin[0, i].item() - math.sin(ang)) < 1e-5
    x = torch.zeros(1, 1, d)
    x[0, 0, 1] = 1.0                                     # only the first element of pair 1
    out = plain.apply_rope_concat_layout(x, cos, sin)[0, 0]
    ang = p * theta ** (-2.0 / d)
    expect = torch.zeros(d)
    expect[1], expect[1 + d // 2] = math.cos(ang), math.sin(ang)
    assert torch.allclose(out, expect, atol=1e-6)


def test_rope_scores_depend_on_distance_only_and_layouts_agree():
    torch.manual_seed(2)
    q, k = torch.randn(1, 2, 32), torch.randn(1, 2, 32)

    def score(m, n, apply):
        cm, sm = plain.rope_cos_sin(torch.tensor([m]), 32, 1e6)
        cn, sn = plain.rope_cos_sin(torch.tensor([n]), 32, 1e6)
        return (apply(q, cm, sm) * apply(k, cn, sn)).sum(-1)

    a = score(3, 1, plain.apply_rope_concat_layout)
    b = score(103, 101, plain.apply_rope_concat_layout)
    assert torch.allclose(a, b, atol=1e-4)                       # a shift of all positions changes nothing
    assert not torch.allclose(a, score(3, 2, plain.apply_rope_concat_layout), atol=1e-3)
    # the reference interleaves the output halves (ullm/layers/rotary_embedding.py:24); q.k is the same
    assert torch.allclose(a, score(3, 1, plain.apply_rope_reference_layout), atol=1e-5)
    # norm of every pair is kept
    c, s = plain.rope_cos_sin(torch.tensor([9]), 32, 1e6)
    r = plain.apply_rope_concat_layout(q, c, s)
    assert torch.allclose(q[..., :16] ** 2 + q[..., 16:] ** 2, r[..., :16] ** 2 + r[..., 16:] ** 2, atol=1e-5)


def test_attention_is_library_attention_with_repeated_kv_heads():
    torch.manual_seed(3)
    T, nq, nkv, d = 9, 6, 2, 16
    q, k, v = torch.randn(T, nq, d), torch.randn(T, nkv, d), torch.randn(T, nkv, d)
    got = plain.causal_gqa_attention(q, k, v, d ** -0.5)
    kr, vr = k.repeat_interleave(nq // nkv, dim=1), v.repeat_interleave(nq // nkv, dim=1)   # head h -> kv h // 3
    ref = F.scaled_dot_product_attention(q.transpose(0, 1), kr.transpose(0, 1), vr.transpose(0, 1), is_causal=True)
    assert torch.allclose(got, ref.transpose(0, 1), atol=1e-5)
    # the wrong group mapping (h % nkv) must differ
    kw, vw = k.repeat(1, nq // nkv, 1), v.repeat(1, nq // nkv, 1)
    wrong = F.scaled_dot_product_attention(q.transpose(0, 1), kw.transpose(0, 1), vw.transpose(0, 1), is_causal=True)
    assert not torch.allclose(got, wrong.transpose(0, 1), atol=1e-3)


def test_attention_special_cases():
    torch.manual_seed(4)
    d = 8
    q, k, v = torch.randn(1, 1, d), torch.randn(1, 1, d), torch.randn(1, 1, d)
    assert torch.allclose(plain.causal_gqa_attention(q, k, v, 1.0), v)          # one token: the value row
    T = 6
    v = torch.randn(T, 1, d)
    out = plain.causal_gqa_attention(torch.zeros(T, 1, d), torch.randn(T, 1, d), v, 1.0)
    for i in range(T):                                                          # equal scores: running mean
        assert torch.allclose(out[i, 0], v[:i + 1, 0].mean(0), atol=1e-6)
    # window w: query i reads keys i-w+1 .. i
    out = plain.causal_gqa_attention(torch.zeros(T, 1, d), torch.randn(T, 1, d), v, 1.0, window=3)
    for i in range(T):
        assert torch.allclose(out[i, 0], v[max(0, i - 2):i + 1, 0].mean(0), atol=1e-6)


def test_silu_and_mul():
    torch.manual_seed(5)
    x = torch.randn(4, 20)
    assert torch.allclose(plain.silu_and_mul(x), F.silu(x[:, :10]) * x[:, 10:])
    x[:, :10] = 0
    assert torch.all(plain.silu_and_mul(x) == 0)                                # zero gate -> zero


def test_whole_model_structure(plain_models):
    """Properties that a norm in the wrong place, a missing residual or a non-causal mix would break."""
    cfg, w = plain_models["B"]
    toks = [5, 400, 17, 3, 250, 99, 1, 77]
    full = plain.qwen3_forward(w, cfg, toks)
    assert full.shape == (8, 503)
    # causal: logits at position i do not depend on later tokens
    assert torch.allclose(plain.qwen3_forward(w, cfg, toks[:5]), full[:5], atol=1e-5)
    # zero all branch outputs: logits = norm(embedding) @ head, the residual path alone
    w0 = dict(w)
    for k in w:
        if k.endswith("o_proj.weight") or k.endswith("down_proj.weight"):
            w0[k] = torch.zeros_like(w[k])
    expect = plain.rms_norm(w["model.embed_tokens.weight"].float()[toks], w["model.norm.weight"], cfg["rms_norm_eps"]) \
        @ w["lm_head.weight"].float().T
    assert torch.allclose(plain.qwen3_forward(w0, cfg, toks), expect, atol=1e-5)
    # q/k norm comes before the rotation and has one gain for all heads: scaling q_proj leaves logits unchanged
    ws = dict(w)
    for k in w:
        if k.endswith("q_proj.weight"):
            ws[k] = w[k].float() * 3.0
    assert torch.allclose(plain.qwen3_forward(ws, cfg, toks), full, atol=2e-4)


def test_tied_head_and_window_option(plain_models):
    cfg, w = plain_models["A"]
    assert "lm_head.weight" not in w
    out = plain.qwen3_forward(w, cfg, [1, 2, 3])
    w2 = dict(w, **{"lm_head.weight": w["model.embed_tokens.weight"]})
    assert torch.equal(out, plain.qwen3_forward(w2, dict(cfg, tie_word_embeddings=False), [1, 2, 3]))
    cfg_c, w_c = plain_models["C"]
    toks = list(range(40))
    with_window = plain.qwen3_forward(w_c, cfg_c, toks)
    without = plain.qwen3_forward(w_c, dict(cfg_c, use_sliding_window=False), toks)
    assert torch.allclose(with_window[:24], without[:24], atol=1e-5)            # the window is not reached yet
    assert not torch.allclose(with_window[30:], without[30:], atol=1e-4)


def test_sampler_reductions():
    torch.manual_seed(6)
    logits = torch.randn(50) * 2
    top = int(logits.argmax())
    assert plain.sample_token(logits, 0.0, -1, 1.0, 0.0, 1, 1) == top
    for kw in (dict(top_k=1, top_p=1.0, min_p=0.0), dict(top_k=-1, top_p=1e-6, min_p=0.0),
               dict(top_k=-1, top_p=1.0, min_p=1.0)):
        for seed in range(5):
            assert plain.sample_token(logits, 1.0, kw["top_k"], kw["top_p"], kw["min_p"], seed, 3) == top
    assert plain.sample_token(logits, 1e-4, -1, 1.0, 0.0, 9, 9) == top          # T -> 0
    # top_k=V, top_p=1, min_p=0: plain softmax sampling; frequencies follow the probabilities
    probs = torch.softmax(logits[:6], -1)
    counts = torch.zeros(6)
    n = 4000
    for pos in range(n):
        counts[plain.sample_token(logits[:6], 1.0, 6, 1.0, 0.0, 1234, pos)] += 1
    chi2 = float(((counts - n * probs) ** 2 / (n * probs)).sum())
    assert chi2 < 25.0, chi2                                                   # 5 degrees of freedom
    # filters: top-k keeps ties, top-p keeps the smallest set whose mass reaches p
    x = plain.filter_logits(torch.tensor([1.0, 3.0, 3.0, 0.0, 2.0]), 1.0, 2, 1.0, 0.0)
    assert torch.isinf(x).tolist() == [True, False, False, True, True]
    x = plain.filter_logits(torch.log(torch.tensor([0.5, 0.3, 0.15, 0.05])), 1.0, -1, 0.8, 0.0)
    assert torch.isinf(x).tolist() == [False, False, True, True]
    x = plain.filter_logits(torch.log(torch.tensor([0.5, 0.3, 0.15, 0.05])), 1.0, -1, 1.0, 0.31)
    assert torch.isinf(x).tolist() == [False, False, True, True]               # 0.15 < 0.31 * 0.5


def test_uniform_is_reproducible_and_spread():
    us = [plain.uniform_from_seed(7, p) for p in range(2000)]
    assert us == [plain.uniform_from_seed(7, p) for p in range(2000)]
    assert all(0.0 <= u < 1.0 for u in us) and abs(sum(us) / 2000 - 0.5) < 0.03
    assert us[:5] != [plain.uniform_from_seed(8, p) for p in range(5)]


# ------------------------------------------------------------------------------------------------
# Pins of the formulas that the reference's text alone fixed before: each is a property of the
# operation itself (an invariant or a special case that is a library routine) that the plausible
# wrong reading does not have.  The reference ships no vectors, and model code of installed packages
# is not a source for this build, so a run of another implementation does not stand here: what these
# cannot reach (the sliding window, which the reference never applies) stays "parity unpinned".

def _attention_weights(cfg, seed, gain_spread=0.0):
    g = torch.Generator().manual_seed(seed)
    nq, nkv, d, H = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"], cfg["hidden_size"]
    rnd = lambda *s: torch.randn(*s, generator=g) * 0.3   # noqa: E731
    w = {"a.q_proj.weight": rnd(nq * d, H), "a.k_proj.weight": rnd(nkv * d, H), "a.v_proj.weight": rnd(nkv * d, H),
         "a.o_proj.weight": rnd(H, nq * d),
         "a.q_norm.weight": 1.0 + gain_spread * torch.rand(d, generator=g),
         "a.k_norm.weight": 1.0 + gain_spread * torch.rand(d, generator=g)}
    return w, rnd


def test_qk_norm_comes_before_the_rotation():
    """Rotary scores depend on the distance of two positions only.  That survives a per-dimension gain
    applied *before* the rotation (it is part of the vectors that are rotated) and not one applied after
    it, unless both halves of every rotated pair have the same gain.  With gains that differ within the
    pairs, shifting all positions must leave the layer's output unchanged: a rotation before the norm's
    gain fails this (checked below on a deliberately swapped copy)."""
    cfg = dict(TINY_B, attention_bias=False)
    w, rnd = _attention_weights(cfg, 11, gain_spread=3.0)
    x = rnd(7, cfg["hidden_size"])
    base = plain.qwen3_attention(x, torch.arange(7), w, "a", cfg, 0)
    shifted = plain.qwen3_attention(x, torch.arange(7) + 40, w, "a", cfg, 0)
    assert torch.allclose(base, shifted, atol=2e-4 * float(base.abs().max()))

    def swapped(x, positions):                      # rotation first, then the per-head norm: the wrong order
        nq, nkv, d, T = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"], x.shape[0]
        q = plain.linear(x, w["a.q_proj.weight"]).view(T, nq, d)
        k = plain.linear(x, w["a.k_proj.weight"]).view(T, nkv, d)
        v = plain.linear(x, w["a.v_proj.weight"]).view(T, nkv, d)
        cos, sin = plain.rope_cos_sin(positions, d, cfg["rope_theta"])
        q = plain.rms_norm(plain.apply_rope_concat_layout(q, cos, sin), w["a.q_norm.weight"], cfg["rms_norm_eps"])
        k = plain.rms_norm(plain.apply_rope_concat_layout(k, cos, sin), w["a.k_norm.weight"], cfg["rms_norm_eps"])
        return plain.linear(plain.causal_gqa_attention(q, k, v, d ** -0.5).reshape(T, nq * d), w["a.o_proj.weight"])
    a, b = swapped(x, torch.arange(7)), swapped(x, torch.arange(7) + 40)
    assert float((a - b).abs().max()) > 1e-2 * float(a.abs().max())     # the invariant tells the two orders apart


def test_attention_layer_without_rotation_is_the_library_routine_with_its_default_scale():
    """With a rotation base so large that every pair but the first stands still, and the first pair's
    gain zero, the layer is projection, per-head RMS norm, plain causal attention, projection.  The
    library routine's default scale is 1/sqrt(size of a query vector) = head_dim^-0.5; here head_dim
    (32) is not hidden_size / heads (12), so a scale taken from the width fails."""
    cfg = dict(TINY_B, attention_bias=False, rope_theta=1e300)
    nq, nkv, d, H = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"], cfg["hidden_size"]
    assert d != H // nq
    w, rnd = _attention_weights(cfg, 12, gain_spread=1.0)
    for n in ("a.q_norm.weight", "a.k_norm.weight"):
        w[n][0] = 0.0
        w[n][d // 2] = 0.0                           # the only pair that still turns (its frequency is 1)
    T = 9
    x = rnd(T, H)
    got = plain.qwen3_attention(x, torch.arange(T) + 5, w, "a", cfg, 0)
    q = F.rms_norm((x @ w["a.q_proj.weight"].T).view(T, nq, d), (d,), w["a.q_norm.weight"], cfg["rms_norm_eps"])
    k = F.rms_norm((x @ w["a.k_proj.weight"].T).view(T, nkv, d), (d,), w["a.k_norm.weight"], cfg["rms_norm_eps"])
    v = (x @ w["a.v_proj.weight"].T).view(T, nkv, d)
    o = F.scaled_dot_product_attention(q.transpose(0, 1)[None], k.transpose(0, 1)[None], v.transpose(0, 1)[None],
                                       is_causal=True, enable_gqa=True)[0].transpose(0, 1)
    want = o.reshape(T, nq * d) @ w["a.o_proj.weight"].T
    assert torch.allclose(got, want, atol=1e-5 * float(want.abs().max()) + 1e-6)
    wrong = F.scaled_dot_product_attention(q.transpose(0, 1)[None], k.transpose(0, 1)[None], v.transpose(0, 1)[None],
                                           is_causal=True, enable_gqa=True, scale=(H // nq) ** -0.5)[0].transpose(0, 1)
    assert not torch.allclose(wrong.reshape(T, nq * d) @ w["a.o_proj.weight"].T, want, atol=1e-3 * float(want.abs().max()))


def test_the_gate_is_the_half_that_goes_through_the_activation():
    """silu(gate) * up is linear in up and not in gate: doubling up_proj doubles the output, doubling
    gate_proj does not.  A feed-forward that activated the other half fails both."""
    g = torch.Generator().manual_seed(13)
    H, I = 24, 40
    w = {"m.gate_proj.weight": torch.randn(I, H, generator=g), "m.up_proj.weight": torch.randn(I, H, generator=g),
         "m.down_proj.weight": torch.randn(H, I, generator=g)}
    x = torch.randn(5, H, generator=g)
    y = plain.qwen3_mlp(x, w, "m")
    y_up = plain.qwen3_mlp(x, dict(w, **{"m.up_proj.weight": 2 * w["m.up_proj.weight"]}), "m")
    y_gate = plain.qwen3_mlp(x, dict(w, **{"m.gate_proj.weight": 2 * w["m.gate_proj.weight"]}), "m")
    assert torch.allclose(y_up, 2 * y, atol=1e-4 * float(y.abs().max()))
    assert float((y_gate - 2 * y).abs().max()) > 1e-2 * float(y.abs().max())
    # and it is the library's activation on that half: one hidden unit, up = 1
    one = {"m.gate_proj.weight": torch.tensor([[1.0]]), "m.up_proj.weight": torch.tensor([[0.0]]),
           "m.down_proj.weight": torch.tensor([[1.0]])}
    t = torch.linspace(-4, 4, 9)[:, None]
    assert torch.all(plain.qwen3_mlp(t, one, "m") == 0)                                          # up = 0 kills it
    one["m.up_proj.weight"] = torch.tensor([[1.0]])
    assert torch.allclose(plain.qwen3_mlp(t, one, "m"), F.silu(t) * t, atol=1e-6)


def test_each_norm_feeds_its_own_branch_and_nothing_else(plain_models):
    """input_layernorm is what attention reads, post_attention_layernorm what the feed-forward reads,
    and neither touches the residual stream: a zero gain on one silences exactly that branch (there are
    no biases), so the model equals the one whose branch output matrix is zero.  A norm placed on a
    branch's output, or on the stream, fails."""
    cfg, w = plain_models["B"]
    toks = [9, 400, 1, 33, 250, 7, 100]
    for layer in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{layer}"
        for norm, out_matrix in ((f"{p}.input_layernorm.weight", f"{p}.self_attn.o_proj.weight"),
                                 (f"{p}.post_attention_layernorm.weight", f"{p}.mlp.down_proj.weight")):
            silenced = plain.qwen3_forward(dict(w, **{norm: torch.zeros_like(w[norm])}), cfg, toks)
            removed = plain.qwen3_forward(dict(w, **{out_matrix: torch.zeros_like(w[out_matrix])}), cfg, toks)
            full = plain.qwen3_forward(w, cfg, toks)
            assert torch.allclose(silenced, removed, atol=1e-5 * float(full.abs().max()))
            assert float((silenced - full).abs().max()) > 1e-3 * float(full.abs().max())
    # pre-norm: the stream itself is never normalised, so scaling the embedding by 1000 makes the branches
    # (whose inputs are normalised) negligible beside it: logits approach norm(embedding) @ head
    big = dict(w, **{"model.embed_tokens.weight": w["model.embed_tokens.weight"].float() * 1000.0})
    expect = plain.rms_norm(w["model.embed_tokens.weight"].float()[toks], w["model.norm.weight"], 0.0) @ w["lm_head.weight"].float().T
    got = plain.qwen3_forward(big, cfg, toks)
    assert float((got - expect).abs().max()) < 2e-2 * float(expect.abs().max())


def test_window_special_cases(plain_models):
    """What can be said of the window without the reference (which has none): a window that reaches the
    start changes nothing, and with a window of one a layer's attention is its own value row."""
    cfg, w = plain_models["C"]
    toks = list(range(30, 60))
    wide = plain.qwen3_forward(w, dict(cfg, sliding_window=len(toks)), toks)
    none = plain.qwen3_forward(w, dict(cfg, use_sliding_window=False), toks)
    assert torch.allclose(wide, none, atol=1e-6)
    torch.manual_seed(14)
    q, k, v = torch.randn(6, 2, 8), torch.randn(6, 2, 8), torch.randn(6, 2, 8)
    assert torch.allclose(plain.causal_gqa_attention(q, k, v, 1.0, window=1), v, atol=1e-6)

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

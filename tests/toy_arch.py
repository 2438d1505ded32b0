"""A test-only architecture, registered from outside the framework: a stack whose layers are chosen
one by one in the config (attention with any position encoding, window, norm and bias option, a
toy mixer with per-request state of fixed size, or a toy mixer that keeps one row per token in pages and
plans its own work lists; a dense feed-forward or a toy one that routes every
token to one of several experts; a toy position encoding with angles of its own), with an optional
run order that names a layer twice or lets a layer read another layer's cache.  Beside it, its plain whole-sequence forward.
Nothing here is a model of anyone's; it exists to show that the framework's parts, cache manager and
step function take new parts without a change to the framework's files."""
from typing import Dict, List

import numpy as np
import torch

import plain_qwen3 as plain
from ullm_amd.models import Choice, ModelPlan, register_architecture
from ullm_amd.kernels import ops
from ullm_amd.parts import (Block, CacheRows, FeedForward, KVNeed, Mixer, PositionEncoding, StateNeed, StepPlan, StepShape,
                            WeightDecl, register_part)
from ullm_amd.parts.linear import linear


@register_part("mixer", "toy_running_mean")
class RunningMean(Mixer):
    """y_t = W * mean(x_0 .. x_t).  State per request: the running sum [hidden] and the count [1],
    kept in float32; a portion continues from the state the previous portion left."""

    def __init__(self, hidden_size: int, prefix: str):
        self.hidden_size, self.prefix = hidden_size, prefix
        self.w = None

    def cache_need(self):
        # a step of single tokens takes the slots from the device (below), so it may be captured
        return StateNeed((self.hidden_size + 1,), torch.float32, graph_safe=True)

    def weights(self):
        return [WeightDecl(f"{self.prefix}.mean_proj.weight", (self.hidden_size, self.hidden_size))]

    def bind(self, tensors, env):
        self.w = tensors[f"{self.prefix}.mean_proj.weight"].contiguous()

    def forward(self, x, ctx, cache):
        H = self.hidden_size
        if ctx.decode_only:
            # one token per entry, token i = entry i: gather the entries' rows, move them on, scatter them
            # back (the padding entries of a captured batch all name the spare row)
            slots = ctx.entry_slot.long()
            rows = cache.state[slots]
            sums, counts = rows[:, :H] + x.float(), rows[:, H] + 1.0
            if cache.owner:
                cache.state[slots] = torch.cat((sums, counts[:, None]), dim=1)
            return linear((sums / counts[:, None]).to(x.dtype), self.w)
        means = torch.empty(x.shape, dtype=torch.float32, device=x.device)
        t = 0
        for n, slot in zip(ctx.host["lens"], ctx.host["slots"]):
            state = cache.state[slot]
            sums = state[:H] + torch.cumsum(x[t:t + n].float(), dim=0)
            counts = state[H] + torch.arange(1, n + 1, device=x.device, dtype=torch.float32)
            means[t:t + n] = sums / counts[:, None]
            if cache.owner:
                state[:H] = sums[-1]
                state[H] = counts[-1]
            t += n
        return linear(means.to(x.dtype), self.w)


def plan_spans(shape: StepShape) -> StepPlan:
    """The work list of the keys-only mixer below, made by the step function through the planner hook: one
    (first token, tokens, keys before them) triple per entry, in batch order."""
    spans, t0 = [], 0
    for n, start in zip(shape.lens, shape.starts):
        spans += [t0, n, start]
        t0 += n
    return StepPlan(arrays={"spans": np.asarray(spans, dtype=np.int32)}, facts={"count": len(shape.lens)})


@register_part("mixer", "toy_keys_only")
class KeysOnly(Mixer):
    """One head whose keys are also its values: y_t = Wo * sum_j softmax_j(q_t . k_j / sqrt(d)) k_j over j <= t.
    It keeps a single row of ``dim`` values per token, in float32 whatever the compute dtype, and says so in
    its need: the step function then allocates that one pool and no value pool.  Its work list comes from a
    planner of its own, named in ``step_planners``."""
    graph_safe = False          # it reads its work list on the host
    step_planners = {"toy_spans": plan_spans}

    def __init__(self, hidden_size: int, dim: int, prefix: str):
        self.hidden_size, self.dim, self.prefix = hidden_size, dim, prefix

    def cache_need(self):
        return KVNeed(1, self.dim, rows=(CacheRows("latent", 1, self.dim, dtype=torch.float32),))

    def weights(self):
        p, H, d = self.prefix, self.hidden_size, self.dim
        return [WeightDecl(f"{p}.q.weight", (d, H)), WeightDecl(f"{p}.k.weight", (d, H)), WeightDecl(f"{p}.o.weight", (H, d))]

    def bind(self, tensors, env):
        p = self.prefix
        self.wq, self.wk, self.wo = (tensors[f"{p}.{n}.weight"].contiguous() for n in ("q", "k", "o"))

    def forward(self, x, ctx, cache):
        d = self.dim
        group = ctx.groups[cache.group]
        pool, P = cache.pools["latent"], group.page_size            # [pages, 1, page_size, dim] float32
        q, k = linear(x, self.wq).float(), linear(x, self.wk).float()
        if cache.owner:
            page = group.block_table[ctx.token_entry.long(), (ctx.positions // P).long()].long()
            pool[page, 0, (ctx.positions % P).long()] = k
        plan = ctx.plans["toy_spans"]
        spans = plan.arrays["spans"].view(-1, 3).tolist()
        assert len(spans) == plan.facts["count"] == ctx.num_entries
        out = torch.empty_like(q)
        for b, (first, n, start) in enumerate(spans):
            total = start + n
            pages = group.block_table[b, :-(-total // P)].long()
            keys = pool[pages, 0].reshape(-1, d)[:total]
            scores = (q[first:first + n] @ keys.T) * d ** -0.5
            seen = torch.arange(total, device=x.device)[None, :] <= (start + torch.arange(n, device=x.device))[:, None]
            out[first:first + n] = torch.softmax(scores.masked_fill(~seen, float("-inf")), dim=-1) @ keys
        return linear(out.to(x.dtype), self.wo)


@register_part("ffn", "toy_top1_experts")
class Top1Experts(FeedForward):
    """Every token goes to the one expert its router scores highest (scores in float32, first index
    on ties); y = softmax(scores)[e] * down_e(relu(up_e x)).  Tokens are gathered per expert, run
    through the framework's linear, and scattered back."""
    graph_safe = False      # each expert gathers the rows routed to it: sizes that depend on the tokens

    def __init__(self, hidden_size: int, expert_size: int, num_experts: int, prefix: str):
        self.hidden_size, self.expert_size, self.num_experts, self.prefix = hidden_size, expert_size, num_experts, prefix

    def weights(self):
        p, H, F = self.prefix, self.hidden_size, self.expert_size
        out = [WeightDecl(f"{p}.router.weight", (self.num_experts, H), keep_fp32=True)]
        for e in range(self.num_experts):
            out += [WeightDecl(f"{p}.experts.{e}.up.weight", (F, H)), WeightDecl(f"{p}.experts.{e}.down.weight", (H, F))]
        return out

    def bind(self, tensors, env):
        p = self.prefix
        self.router = tensors[f"{p}.router.weight"]
        self.up = [tensors[f"{p}.experts.{e}.up.weight"].contiguous() for e in range(self.num_experts)]
        self.down = [tensors[f"{p}.experts.{e}.down.weight"].contiguous() for e in range(self.num_experts)]

    def forward(self, x, ctx):
        scores = x.float() @ self.router.float().T
        choice = scores.argmax(dim=-1)
        weight = torch.softmax(scores, dim=-1).gather(1, choice[:, None])
        out = torch.zeros(x.shape, dtype=torch.float32, device=x.device)
        for e in range(self.num_experts):
            rows = torch.nonzero(choice == e).flatten()
            if rows.numel():
                hidden = torch.relu(linear(x[rows].contiguous(), self.up[e]))
                out[rows] = linear(hidden, self.down[e]).float()
        return (out * weight).to(x.dtype)


@register_part("position", "toy_linear_angles")
class LinearAngles(PositionEncoding):
    """Adjacent pairs rotated by angle[p, i] = p * step * (i + 1): another table for the same kernel."""

    def __init__(self, head_dim: int, step: float):
        self.head_dim, self.step = head_dim, float(step)
        self.table = None

    @staticmethod
    def angles(positions: torch.Tensor, head_dim: int, step: float) -> torch.Tensor:
        return positions.to(torch.float32)[:, None] * (step * torch.arange(1, head_dim // 2 + 1, dtype=torch.float32))[None, :]

    def bind(self, tensors, env):
        a = self.angles(torch.arange(env.context_len), self.head_dim, self.step)
        self.table = torch.cat((a.cos(), a.sin()), dim=-1).contiguous().to(env.device)

    def kernel_args(self):
        return self.table, self.head_dim, 2


@register_part("block", "toy_two_mixers")
class TwoMixers(Block):
    """h += attention(norm1 h) + running_mean(norm1 h); h += ffn(norm2 h).  One block that keeps keys
    and values *and* fixed-size state: it declares both needs and hands each mixer its own view."""

    def __init__(self, mixer_norm, attention, mean, ffn_norm, ffn):
        self.mixer_norm, self.attention, self.mean, self.ffn_norm, self.ffn = mixer_norm, attention, mean, ffn_norm, ffn

    def children(self):
        return [self.mixer_norm, self.attention, self.mean, self.ffn_norm, self.ffn]

    def cache_need(self):
        return [self.attention.cache_need(), self.mean.cache_need()]

    def forward(self, residual, pending, ctx, cache):
        x = self.mixer_norm.add_norm(pending, residual, out_dtype=ctx.dtype)
        kv_view, state_view = cache.parts
        a = self.attention.forward(x, ctx, kv_view)
        if a.dim() == 3:                       # a stack of partial sums: this block adds them itself
            a = a.sum(0)
        ops.residual_add(a.contiguous(), residual)
        pending = self.mean.forward(x, ctx, state_view)
        return residual, self.ffn.forward(self.ffn_norm.add_norm(pending, residual, out_dtype=ctx.dtype), ctx)


def toy_config_from_dict(d):
    return dict(d)


def toy_plan(cfg: dict) -> ModelPlan:
    H, eps = cfg["hidden_size"], cfg["eps"]
    layers = []
    for i, L in enumerate(cfg["layers"]):
        p = f"stack.{i}"
        if L["mixer"] in ("attention", "both"):
            rope = L.get("rope", "half")
            if rope == "none":
                position = None
            elif rope == "toy_linear":
                position = Choice("position", "toy_linear_angles", dict(head_dim=L["head_dim"], step=L["angle_step"]))
            else:
                position = Choice("position", "rotary", dict(
                    head_dim=L["head_dim"], theta=cfg["theta"], rotary_dim=L.get("rotary_dim", L["head_dim"]), pairing=rope))
            mixer = Choice("mixer", "gqa_attention", dict(
                hidden_size=H, num_heads=L["heads"], num_kv_heads=L["kv_heads"], head_dim=L["head_dim"],
                prefix=f"{p}.attn", position=position, qk_norm_eps=eps if L.get("qk_norm", True) else None,
                bias=L.get("bias", False), window=L.get("window", 0), scale=L.get("scale")))
        elif L["mixer"] == "keys_only":
            mixer = Choice("mixer", "toy_keys_only", dict(hidden_size=H, dim=L["dim"], prefix=f"{p}.lat"))
        else:
            mixer = Choice("mixer", "toy_running_mean", dict(hidden_size=H, prefix=f"{p}.mix"))
        norm = lambda n: Choice("norm", "rmsnorm", dict(size=H, eps=eps, weight_name=f"{p}.{n}.weight"))  # noqa: E731
        if L.get("experts"):
            ffn = Choice("ffn", "toy_top1_experts", dict(hidden_size=H, expert_size=L["ffn_size"],
                                                         num_experts=L["experts"], prefix=f"{p}.ffn"))
        else:
            ffn = Choice("ffn", "swiglu", dict(hidden_size=H, intermediate_size=L["ffn_size"], prefix=f"{p}.ffn"))
        if L["mixer"] == "both":
            mean = Choice("mixer", "toy_running_mean", dict(hidden_size=H, prefix=f"{p}.mix"))
            layers.append(Choice("block", "toy_two_mixers", dict(
                mixer_norm=norm("norm1"), attention=mixer, mean=mean, ffn_norm=norm("norm2"), ffn=ffn)))
            continue
        layers.append(Choice("block", "prenorm", dict(
            mixer_norm=norm("norm1"), mixer=mixer, ffn_norm=norm("norm2"), ffn=ffn)))
    order = [tuple(x) for x in cfg["run_order"]] if cfg.get("run_order") else None
    return ModelPlan(vocab_size=cfg["vocab_size"], hidden_size=H, embedding_weight="tok.weight", layers=layers,
                     final_norm=Choice("norm", "rmsnorm", dict(size=H, eps=eps, weight_name="out_norm.weight")),
                     head_weight="head.weight", tie_head_to_embedding=cfg.get("tie", False), run_order=order,
                     init_std=cfg.get("init_std", 0.05), embedding_scale=cfg.get("embed_scale", 1.0),
                     head_bias="head.bias" if cfg.get("head_bias") else None, logit_softcap=cfg.get("logit_cap", 0.0))


register_architecture("ToyStackForCausalLM", toy_config_from_dict, toy_plan)


# ---------------------------------------------------------------------------------------- plain forward

def _rope(x, positions, L, theta):
    rope = L.get("rope", "half")
    if rope == "none":
        return x
    rot = L.get("rotary_dim", L["head_dim"])
    if rope == "toy_linear":
        a = LinearAngles.angles(positions, L["head_dim"], L["angle_step"])
        cos, sin = a.cos(), a.sin()
    else:
        cos, sin = plain.rope_cos_sin(positions, rot, theta)
    r, rest = x[..., :rot], x[..., rot:]
    if rope == "half":
        r = plain.apply_rope_concat_layout(r, cos, sin)
    else:
        a, b = r[..., 0::2], r[..., 1::2]
        c, s = cos.unsqueeze(1), sin.unsqueeze(1)
        r = torch.stack((a * c - b * s, b * c + a * s), -1).flatten(-2)
    return torch.cat((r, rest), -1)


def toy_forward(w: Dict[str, torch.Tensor], cfg: dict, token_ids: List[int]) -> torch.Tensor:
    w = {k: v.float() for k, v in w.items()}
    T, eps = len(token_ids), cfg["eps"]
    positions = torch.arange(T)
    h = w["tok.weight"][torch.tensor(token_ids)] * cfg.get("embed_scale", 1.0)
    order = cfg.get("run_order") or [[i, i] for i in range(len(cfg["layers"]))]
    kv_of: Dict[int, tuple] = {}
    for layer, cache_id in order:
        L, p = cfg["layers"][layer], f"stack.{layer}"
        x = plain.rms_norm(h, w[f"{p}.norm1.weight"], eps)
        a = 0.0
        if L["mixer"] in ("attention", "both"):
            nq, nkv, d = L["heads"], L["kv_heads"], L["head_dim"]
            b = (lambda n: w[f"{p}.attn.{n}_proj.bias"]) if L.get("bias", False) else (lambda n: None)
            q = plain.linear(x, w[f"{p}.attn.q_proj.weight"], b("q")).view(T, nq, d)
            if L.get("qk_norm", True):
                q = plain.rms_norm(q, w[f"{p}.attn.q_norm.weight"], eps)
            q = _rope(q, positions, L, cfg["theta"])
            if cache_id not in kv_of:                     # the first layer that names a cache writes it
                k = plain.linear(x, w[f"{p}.attn.k_proj.weight"], b("k")).view(T, nkv, d)
                v = plain.linear(x, w[f"{p}.attn.v_proj.weight"], b("v")).view(T, nkv, d)
                if L.get("qk_norm", True):
                    k = plain.rms_norm(k, w[f"{p}.attn.k_norm.weight"], eps)
                kv_of[cache_id] = (_rope(k, positions, L, cfg["theta"]), v)
            k, v = kv_of[cache_id]
            scale = L.get("scale") or d ** -0.5
            o = plain.causal_gqa_attention(q, k, v, scale, L.get("window", 0))
            a = plain.linear(o.reshape(T, nq * d), w[f"{p}.attn.o_proj.weight"])
        if L["mixer"] == "keys_only":
            d = L["dim"]
            q, k = plain.linear(x, w[f"{p}.lat.q.weight"]), plain.linear(x, w[f"{p}.lat.k.weight"])
            if cache_id not in kv_of:
                kv_of[cache_id] = (k, k)
            k = kv_of[cache_id][0]
            o = plain.causal_gqa_attention(q.view(T, 1, d), k.view(T, 1, d), k.view(T, 1, d), d ** -0.5)
            a = plain.linear(o.reshape(T, d), w[f"{p}.lat.o.weight"])
        elif L["mixer"] != "attention":
            means = torch.cumsum(x, 0) / torch.arange(1, T + 1, dtype=torch.float32)[:, None]
            a = a + plain.linear(means, w[f"{p}.mix.mean_proj.weight"])
        h = h + a
        x = plain.rms_norm(h, w[f"{p}.norm2.weight"], eps)
        if L.get("experts"):
            scores = x @ w[f"{p}.ffn.router.weight"].T
            probs = torch.softmax(scores, -1)
            y = torch.zeros_like(x)
            for t in range(T):
                e = int(scores[t].argmax())
                hidden = torch.relu(plain.linear(x[t], w[f"{p}.ffn.experts.{e}.up.weight"]))
                y[t] = probs[t, e] * plain.linear(hidden, w[f"{p}.ffn.experts.{e}.down.weight"])
            h = h + y
        else:
            gu = torch.cat((plain.linear(x, w[f"{p}.ffn.gate_proj.weight"]),
                            plain.linear(x, w[f"{p}.ffn.up_proj.weight"])), -1)
            h = h + plain.linear(plain.silu_and_mul(gu), w[f"{p}.ffn.down_proj.weight"])
    x = plain.rms_norm(h, w["out_norm.weight"], eps)
    logits = plain.linear(x, w["head.weight"] if "head.weight" in w else w["tok.weight"], w.get("head.bias"))
    cap = cfg.get("logit_cap", 0.0)
    return cap * torch.tanh(logits / cap) if cap else logits

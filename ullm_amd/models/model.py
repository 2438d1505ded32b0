"""A model as data: which parts make each layer, in which order layers run, whose cache a layer
reads.  ``Model`` builds the parts named by a ``ModelPlan`` from the part registry, collects their
declared weights and cache needs, and runs the layer list over a batch.

Reference shape of the same thing: ullm/models/qwen3.py:199-286 (embedding, layer loop carrying
(hidden, residual), final norm, lm_head on selected rows ullm/core/model_runner.py:339-341).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Sequence, Tuple

import torch

from ..cache.manager import CacheGroupSpec
from ..kernels import ops
from ..parts import (Block, KVNeed, LayerCache, Norm, Part, PartEnv, StateNeed, StepContext, WeightDecl,
                     build_part, cache_needs_of, walk)
from ..parts.linear import linear


@dataclass(frozen=True)
class Choice:
    """A part chosen by name with its parameters; parameters may themselves be choices."""
    kind: str
    name: str
    params: Dict[str, Any] = field(default_factory=dict)

    def build(self) -> Part:
        built = {k: (v.build() if isinstance(v, Choice) else v) for k, v in self.params.items()}
        return build_part(self.kind, self.name, **built)


@dataclass
class ModelPlan:
    vocab_size: int
    hidden_size: int
    embedding_weight: str                    # tensor name of the token table [vocab, hidden]
    layers: List[Choice]                     # one "block" choice per layer
    final_norm: Choice
    head_weight: str                         # tensor name of the output matrix [vocab, hidden]
    tie_head_to_embedding: bool = False      # bind the token table where the head tensor is absent
    embedding_scale: float = 1.0             # the token rows are multiplied by this on their way into the stream
    head_bias: Optional[str] = None          # tensor name of a bias [vocab] on the logits, float32
    logit_softcap: float = 0.0               # > 0: logits = cap * tanh(logits / cap)
    # The order layers run in: (layer, cache id).  A layer may appear more than once (with a cache id
    # of its own each time, or the same one).  The first entry that names a cache id owns that cache
    # and writes it; later entries with the same id only read it, so a layer can read the cache
    # another layer wrote.  Default: every layer once, cache id = layer index.
    run_order: Optional[List[Tuple[int, int]]] = None
    init_std: float = 0.02                   # random-weights mode

    def order(self) -> List[Tuple[int, int]]:
        return self.run_order if self.run_order is not None else [(i, i) for i in range(len(self.layers))]


class Model:
    def __init__(self, plan: ModelPlan):
        self.plan = plan
        self.blocks: List[Block] = [c.build() for c in plan.layers]
        self.final_norm: Norm = plan.final_norm.build()
        self.run_order = plan.order()
        self.cache_owner: Dict[int, int] = {}      # cache id -> index into run_order of its owner
        for idx, (layer, cache_id) in enumerate(self.run_order):
            if not (0 <= layer < len(self.blocks)):
                raise ValueError(f"run order names layer {layer}: out of range")
            self.cache_owner.setdefault(cache_id, idx)
        self.embedding: Optional[torch.Tensor] = None
        self.head: Optional[torch.Tensor] = None
        self.head_bias: Optional[torch.Tensor] = None
        self.env: Optional[PartEnv] = None

    # ------------------------------------------------------------------ weights
    def parts(self):
        for b in self.blocks:
            yield from walk(b)
        yield from walk(self.final_norm)

    def weight_decls(self) -> List[WeightDecl]:
        p = self.plan
        decls = [WeightDecl(p.embedding_weight, (p.vocab_size, p.hidden_size))]
        for part in self.parts():
            decls.extend(part.weights())
        decls.append(WeightDecl(p.head_weight, (p.vocab_size, p.hidden_size),
                                alias_of=p.embedding_weight if p.tie_head_to_embedding else None))
        if p.head_bias:
            decls.append(WeightDecl(p.head_bias, (p.vocab_size,), keep_fp32=True))
        return decls

    def bind(self, tensors: Dict[str, torch.Tensor], env: PartEnv) -> None:
        self.env = env
        self.embedding = tensors[self.plan.embedding_weight].contiguous()
        self.head = tensors[self.plan.head_weight].contiguous()
        self.head_bias = tensors[self.plan.head_bias].contiguous() if self.plan.head_bias else None
        for part in self.parts():
            part.bind(tensors, env)

    # ------------------------------------------------------------------ cache layout
    def cache_layout(self):
        """Groups of caches with equal needs, and the per-request state needs.  A cache is named by
        (cache id, index of the need among those its block declares).
        Returns (groups, {(cache id, need index): group index}, {(cache id, need index): StateNeed})."""
        keyed: Dict[KVNeed, List[Tuple[int, int]]] = {}
        states: Dict[Tuple[int, int], StateNeed] = {}
        for cache_id, idx in self.cache_owner.items():
            for i, need in enumerate(cache_needs_of(self.blocks[self.run_order[idx][0]])):
                if isinstance(need, KVNeed):
                    keyed.setdefault(need, []).append((cache_id, i))
                else:
                    states[(cache_id, i)] = need
        groups, cache_group = [], {}
        for need, keys in keyed.items():
            for c in keys:
                cache_group[c] = len(groups)
            rows = tuple((r.heads, r.dim, None if r.dtype is None else torch.empty((), dtype=r.dtype).element_size())
                         for r in need.rows) if need.rows else None
            groups.append(CacheGroupSpec(need.num_kv_heads, need.head_dim, need.window, tuple(keys), rows))
        self._group_needs = list(keyed)
        for idx, (layer, cache_id) in enumerate(self.run_order):
            owner_layer = self.run_order[self.cache_owner[cache_id]][0]
            a, b = cache_needs_of(self.blocks[layer]), cache_needs_of(self.blocks[owner_layer])
            if a != b:
                raise ValueError(f"layer {layer} reads cache {cache_id} written by layer {owner_layer} "
                                 f"but their needs differ: {a} vs {b}")
        return groups, cache_group, states

    def group_needs(self) -> List[KVNeed]:
        """The paged need of every cache group, in the order of :meth:`cache_layout`'s groups."""
        self.cache_layout()
        return self._group_needs

    def num_needs(self, cache_id: int) -> int:
        """How many needs the block that owns this cache declares."""
        return len(cache_needs_of(self.blocks[self.run_order[self.cache_owner[cache_id]][0]]))

    # ------------------------------------------------------------------ forward
    def forward(self, ctx: StepContext, caches: Dict[int, LayerCache], logit_rows: Optional[torch.Tensor]):
        """Runs the batch through every layer of the run order and returns float32 logits
        [len(logit_rows), vocab] (None if no row is wanted)."""
        residual = ops.embedding(ctx.token_ids, self.embedding, scale=self.plan.embedding_scale)
        pending = None
        for idx, (layer, cache_id) in enumerate(self.run_order):
            cache = caches.get(cache_id)
            if cache is None:
                cache = LayerCache()
            elif self.cache_owner[cache_id] != idx:
                cache = cache.reader()
            block = self.blocks[layer]
            if block.hands_norm_ahead and idx + 1 < len(self.run_order):
                # a block whose last kernel can prepare the norm that follows is told which norm that is
                after = self.blocks[self.run_order[idx + 1][0]].entry_norm()
                residual, pending = block.forward(residual, pending, ctx, cache, next_norm=after)
            else:
                residual, pending = block.forward(residual, pending, ctx, cache)
        if logit_rows is None or logit_rows.numel() == 0:
            return None
        x = self.final_norm.add_norm(pending, residual, rows=logit_rows, out_dtype=ctx.dtype)
        logits = linear(x, self.head, self.head_bias, out_dtype=torch.float32)
        if self.plan.logit_softcap > 0:
            ops.softcap_(logits, self.plan.logit_softcap)
        return logits

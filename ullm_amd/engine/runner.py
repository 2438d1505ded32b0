"""The step function: one batch of (request, its next tokens) through the model, from the cache.

Reference: ullm/core/model_runner.py:298-363 with ullm/core/input_batch.py:80-220.  There a batch
is either whole prompts or one token per request (model_runner.py:309-311) and the step returns
sampled ids only.  Here any mix of prompt portions and single decoded tokens is one batch, cut
anywhere; only the tokens given are run, everything earlier comes from the cache, and the step
returns 32-bit logits at the places asked for.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

from ..cache.manager import CacheManager, RequestCache
from ..kernels import ops
from ..models.model import Model
from ..parts import GroupView, LayerCache, PartEnv, StepContext, StepPlan, StepShape
from ..staging import StagedUpload


@dataclass
class StepEntry:
    """One request's next tokens.  ``want`` lists the places among these tokens whose logits are
    returned (it may be empty)."""
    cache: RequestCache
    tokens: Sequence[int]
    want: Sequence[int] = field(default_factory=list)


class StepError(RuntimeError):
    pass


UNKNOWN_TOKEN = -2         # stands for a token that is still being sampled when the step is prepared


def batch_bucket(n: int) -> int:
    """The batch size of the captured graph that a decode step of ``n`` requests replays: the next power of
    two, or three quarters of it from 48 on (48, 96, 192: whole 16-row tiles, and the projections' cost
    follows the number of such tiles from there on; below, the kernels take 16 or 32 rows at one cost)."""
    b = 1
    while b < n:
        b *= 2
    return b * 3 // 4 if b >= 64 and n <= b * 3 // 4 else b


class ModelRunner:
    def __init__(self, model: Model, env: PartEnv, page_size: int, num_pages, max_requests: int,
                 enable_prefix_cache: bool = False, use_graphs: bool = True, max_graph_batch: int = 256):
        if model.env is None:
            raise StepError("the model has no weights bound")
        self.model, self.env = model, env
        # may mixers and feed-forwards hand the next norm a stack of partial sums?  Only if every norm adds one up
        self._stacked_branches = all(getattr(part, "adds_stacks", False) for part in model.parts() if part.kind == "norm")
        self.page_size = page_size
        self.max_requests = max_requests
        groups, cache_group, states = model.cache_layout()
        if isinstance(num_pages, int):
            num_pages = [num_pages] * len(groups)
        self.cache = CacheManager(groups, list(num_pages), page_size, max_requests,
                                  enable_prefix_cache=enable_prefix_cache and not states)
        self.max_table = -(-env.context_len // page_size)
        views: Dict[tuple, LayerCache] = {}      # (cache id, index of the need in its block) -> view
        for g, (spec, need) in enumerate(zip(groups, model.group_needs())):
            for key in spec.layers:
                pools = {}
                for rows in need.pools():
                    shape = ((num_pages[g], rows.heads, rows.dim, page_size) if rows.transposed
                             else (num_pages[g], rows.heads, page_size, rows.dim))
                    # zeroed once so that no row ever holds a non-finite bit pattern before it is written
                    pools[rows.name] = torch.zeros(shape, dtype=rows.dtype or env.dtype, device=env.device)
                views[key] = LayerCache.of_pools(g, pools)
        for key, need in states.items():
            # one row more than requests: the slot of a captured batch's padding entries
            views[key] = LayerCache(
                state=torch.zeros((max_requests + 1,) + tuple(need.shape), dtype=need.dtype, device=env.device))
        self._views = views
        self._states = [c.state.view(c.state.shape[0], -1) for c in views.values() if c.state is not None]
        # what the parts' kernels want to know about a step beside the flat batch (Part.step_planners)
        self._planners: Dict[str, object] = {}
        for part in model.parts():
            for name, planner in part.step_planners.items():
                if self._planners.setdefault(name, planner) is not planner:
                    raise StepError(f"two parts name different step planners {name!r}")
        # per cache id what its block sees: the one view, or one view per declared need
        self.caches: Dict[int, LayerCache] = {}
        for cache_id in sorted({c for c, _ in views}):
            self.caches[cache_id] = LayerCache.of_parts([views[(cache_id, i)] for i in range(model.num_needs(cache_id))])
        self._upload = StagedUpload(env.device)
        # int32 device tensor the steps take late token ids from (the sampler's output of the step before), or None
        self.feed_source: Optional[torch.Tensor] = None
        self.vocab_size = model.plan.vocab_size
        # Steps in which every entry brings one token are replayed from HIP graphs, one graph per
        # (batch size bucket, context length bucket), unless a part says that its work cannot be captured
        # (Part.graph_safe); with state mixers only if each of them says that its single-token step can be
        # (StateNeed.graph_safe).
        self.use_graphs = (bool(use_graphs) and env.device.type == "cuda"
                           and all(need.graph_safe for need in states.values())
                           and all(part.graph_safe for part in model.parts()))
        self.padding_slot = max_requests
        self.max_graph_batch = max_graph_batch
        self._graphs: Dict[tuple, "_DecodeGraph"] = {}
        self._graph_pool = None

    # ------------------------------------------------------------------ helpers
    def cache_bytes(self) -> int:
        total = 0
        for c in self._views.values():
            for t in list(c.pools.values()) + [c.state]:
                if t is not None:
                    total += t.numel() * t.element_size()
        return total

    def _pack(self, entries: Sequence[StepEntry], pad_entries: int = 0, table_stride: Optional[int] = None,
              allow_unknown: bool = False, kv_bucket: Optional[int] = None):
        """Flatten the entries into one int32 host array.  Returns (host array, layout, facts); the layout
        maps a field's name to its (first, end) in the array.
        ``pad_entries`` > len(entries) appends one-token entries that hold no pages (their cache
        writes are skipped and their outputs ignored), so that a batch fits a captured graph; every entry's
        only token is then a wanted row and ``picked`` lists the entries that asked for it.
        With ``allow_unknown`` a token may be UNKNOWN_TOKEN (its id is filled in before the launch);
        ``facts["unknown"]`` lists such tokens as (index into the array, entry, index in the entry)."""
        P = self.page_size
        n_real = len(entries)
        lens = [len(e.tokens) for e in entries]
        if n_real == 0 or sum(lens) == 0:
            raise StepError("a step needs at least one token")
        n_pad = max(0, pad_entries - n_real)
        for_graph = pad_entries > 0
        B = n_real + n_pad
        T = sum(lens) + n_pad
        groups = self.cache.groups
        strides = []
        for g in range(len(groups)):
            widest = max(1, max(len(e.cache.tables[g]) for e in entries))
            if table_stride is not None:
                if widest > table_stride:
                    raise StepError("a block table is wider than the captured graph's")
                widest = table_stride
            strides.append(widest)
        caches = [e.cache for e in entries]
        starts = [rc.num_computed for rc in caches]
        slots = [rc.slot for rc in caches]
        for rc, n, s0 in zip(caches, lens, starts):
            if n < 1:
                raise StepError(f"request {rc.request_id!r}: an entry needs at least one token")
            if rc.released:
                raise StepError(f"request {rc.request_id!r} was released")
            if s0 + n > self.env.context_len:
                raise StepError(f"request {rc.request_id!r}: {s0 + n} tokens exceed context_len={self.env.context_len}")
            for tab in rc.tables:
                if len(tab) * P < s0 + n:
                    raise StepError(f"request {rc.request_id!r}: no pages reserved for positions up to {s0 + n - 1}")
        if len(set(slots)) != n_real:
            seen = set()
            for rc in caches:
                if rc.slot in seen:
                    raise StepError(f"request {rc.request_id!r} appears twice in one step")
                seen.add(rc.slot)
        picked = [b for b, e in enumerate(entries) if len(e.want)] if for_graph else []
        n_want = B if for_graph else sum(len(e.want) for e in entries)
        shape = StepShape(tuple(lens), tuple(starts), n_pad, kv_bucket)
        plans = {name: planner(shape) for name, planner in self._planners.items()}
        fields = [("ids", T), ("positions", T), ("token_entry", T), ("q_start", B + 1), ("slot", B), ("start", B),
                  ("rows", n_want), ("picked", B if for_graph else 0)]
        fields += [(f"table{g}", B * stride) for g, stride in enumerate(strides)]
        for name, plan in plans.items():
            for key, arr in plan.arrays.items():
                arr = np.asarray(arr)
                if arr.dtype != np.int32 or arr.ndim != 1:
                    raise StepError(f"step planner {name!r}: array {key!r} must be a flat int32 array")
                fields.append((f"plan.{name}.{key}", arr.size))
        fields.append(("feed", T))
        layout, at = {}, 0
        for name, size in fields:
            layout[name] = (at, at + size)
            at += size
        host = np.zeros(at, dtype=np.int32)
        part = lambda name: host[layout[name][0]:layout[name][1]]   # noqa: E731
        ids, pos, ent, q_start, rows = part("ids"), part("positions"), part("token_entry"), part("q_start"), part("rows")
        part("feed")[:] = -1                             # per token: where the device takes its id from (-1: from ids)
        n_tok = T - n_pad
        tok = np.empty(n_tok, dtype=np.int64)
        if n_tok == n_real:                              # one token each: no per-entry array work
            tok[:] = [e.tokens[0] for e in entries]
            pos[:n_real] = starts
            ent[:n_real] = np.arange(n_real)
            q_start[:n_real] = ent[:n_real]
        else:
            first = np.zeros(n_real + 1, dtype=np.int64)
            np.cumsum(lens, out=first[1:])
            q_start[:n_real] = first[:n_real]
            ent[:n_tok] = np.repeat(np.arange(n_real), lens)
            pos[:n_tok] = np.arange(n_tok) - np.repeat(first[:n_real] - np.asarray(starts, dtype=np.int64), lens)
            t = 0
            for e, n in zip(entries, lens):
                tok[t:t + n] = e.tokens
                t += n
        unknown = []
        if allow_unknown and int(tok.min()) == UNKNOWN_TOKEN:
            first_of = q_start[:n_real]
            for t in np.nonzero(tok == UNKNOWN_TOKEN)[0].tolist():
                b = int(ent[t])
                unknown.append((layout["ids"][0] + t, layout["feed"][0] + t, b, t - int(first_of[b])))
            tok[tok == UNKNOWN_TOKEN] = 0
        if int(tok.min()) < 0 or int(tok.max()) >= self.vocab_size:
            bad = next(rc for rc, e in zip(caches, entries) if min(e.tokens) < 0 or max(e.tokens) >= self.vocab_size)
            raise StepError(f"request {bad.request_id!r}: token id outside [0, {self.vocab_size})")
        ids[:n_tok] = tok
        part("slot")[:n_real] = slots
        part("slot")[n_real:] = self.padding_slot
        part("start")[:n_real] = starts
        r = 0
        for b, e in enumerate(entries):
            for w in ([0] if for_graph else e.want):
                if not (0 <= w < lens[b]):
                    raise StepError(f"request {caches[b].request_id!r}: wanted place {w} outside its {lens[b]} tokens")
                rows[r] = q_start[b] + w
                r += 1
        t = n_tok
        for b in range(n_real, B):                       # padding entries: token 0 at position 0, no pages
            ent[t] = b
            q_start[b] = t
            rows[r] = t
            t += 1
            r += 1
        q_start[B] = T
        part("picked")[:len(picked)] = picked
        for g, stride in enumerate(strides):
            bt = part(f"table{g}").reshape(B, stride)
            bt[:n_real] = self.cache.table_rows(g, slots, stride)
            bt[n_real:] = -1
        for name, plan in plans.items():
            for key, arr in plan.arrays.items():
                part(f"plan.{name}.{key}")[:] = arr
        facts = dict(T=T, B=B, strides=strides, n_want=n_want, picked=picked, max_q=max(lens),
                     max_kv=kv_bucket or max(s0 + n for s0, n in zip(starts, lens)),
                     decode_only=all(n == 1 for n in lens), lens=lens + [1] * n_pad,
                     starts=starts + [0] * n_pad, slots=slots + [self.padding_slot] * n_pad, unknown=unknown,
                     plans={name: plan.facts for name, plan in plans.items()},
                     plan_arrays={name: list(plan.arrays) for name, plan in plans.items()})
        return host, layout, facts

    def _context(self, dev: torch.Tensor, layout, facts) -> tuple:
        """Views into the uploaded buffer as a StepContext, and the wanted rows."""
        groups = self.cache.groups
        B, T = facts["B"], facts["T"]
        view = lambda name: dev[layout[name][0]:layout[name][1]]  # noqa: E731
        gviews = [GroupView(view(f"table{g}").view(B, facts["strides"][g]), facts["strides"][g], self.page_size,
                            groups[g].window) for g in range(len(groups))]
        plans = {name: StepPlan({key: view(f"plan.{name}.{key}") for key in facts["plan_arrays"][name]}, dict(numbers))
                 for name, numbers in facts["plans"].items()}
        ctx = StepContext(
            num_tokens=T, num_entries=B, token_ids=view("ids"), positions=view("positions"),
            token_entry=view("token_entry"), q_start=view("q_start"), entry_slot=view("slot"),
            entry_start=view("start"), groups=gviews, max_q_len=facts["max_q"], max_kv_len=facts["max_kv"],
            decode_only=facts["decode_only"], dtype=self.env.dtype, stacked_branches=self._stacked_branches,
            host={"lens": facts["lens"], "starts": facts["starts"], "slots": facts["slots"]}, plans=plans)
        return ctx, (view("rows") if facts["n_want"] else None)

    def _forward(self, dev: torch.Tensor, layout, ctx: StepContext, rows) -> Optional[torch.Tensor]:
        """The device work of a step, the same whether it runs now or is captured: late token ids, the state
        rows of requests that start at their first token zeroed, the model."""
        if self.feed_source is not None:
            ops.feed_tokens(dev[layout["ids"][0]:layout["ids"][1]], dev[layout["feed"][0]:layout["feed"][1]],
                            self.feed_source)
        for state in self._states:
            ops.zero_fresh_rows(state, ctx.entry_slot, ctx.entry_start, ctx.num_entries)
        return self.model.forward(ctx, self.caches, rows)

    # ------------------------------------------------------------------ the step
    def step(self, entries: Sequence[StepEntry]) -> Optional[torch.Tensor]:
        """Run the entries as one batch.  Pages for the new tokens must have been reserved.
        Returns float32 logits [number of wanted places, vocab] in the order of the entries and of
        their ``want`` lists, or None if nothing is wanted.  On return the requests' caches hold the
        new tokens (``num_computed`` has advanced)."""
        return self.launch(self.prepare(entries))

    def prepare(self, entries: Sequence[StepEntry], allow_unknown: bool = False) -> "PreparedStep":
        """The host half of a step: checks and the packed batch description.  Nothing is queued on
        the device, so this may run while an earlier step is still computing; the requests' caches
        must already be in the state in which the step will find them."""
        entries = list(entries)
        if (self.use_graphs and len(entries) <= self.max_graph_batch and all(len(e.tokens) == 1 for e in entries)):
            b_pad = batch_bucket(len(entries))
            longest = max(e.cache.num_computed + 1 for e in entries)
            kv_bucket = 256
            while kv_bucket < longest:
                kv_bucket *= 2
            kv_bucket = min(kv_bucket, self.max_table * self.page_size)
            host, layout, facts = self._pack(entries, pad_entries=b_pad, table_stride=self.max_table,
                                             allow_unknown=allow_unknown, kv_bucket=kv_bucket)
            return PreparedStep(entries, host, layout, facts, (b_pad, kv_bucket))
        host, layout, facts = self._pack(entries, allow_unknown=allow_unknown)
        return PreparedStep(entries, host, layout, facts, None)

    def stage(self, prepared: "PreparedStep") -> None:
        """Copy a prepared step's description into pinned memory ahead of its launch (optional: the
        launch does it otherwise).  Only the step that will be launched next may be staged."""
        prepared.staged = self._upload.stage(prepared.host)

    def _send(self, prepared: "PreparedStep", into: Optional[torch.Tensor] = None) -> torch.Tensor:
        staged = prepared.staged if prepared.staged is not None else self._upload.stage(prepared.host)
        prepared.staged = None
        return self._upload.send(staged, into)

    def launch(self, prepared: "PreparedStep") -> Optional[torch.Tensor]:
        """The device half: upload, the model's kernels (or a graph replay), and the caches' counters."""
        if prepared.facts["unknown"]:
            raise StepError("a prepared step still holds tokens without an id")
        entries = prepared.entries
        if prepared.graph_key is not None:
            logits = self._launch_graph(prepared)
        else:
            dev = self._send(prepared)
            ctx, rows = self._context(dev, prepared.layout, prepared.facts)
            with torch.no_grad():
                logits = self._forward(dev, prepared.layout, ctx, rows)
        for e in entries:
            self.cache.commit(e.cache, len(e.tokens))
        return logits

    def build_context(self, entries: Sequence[StepEntry]):
        """Flatten the entries into device tensors (one host-to-device copy)."""
        host, layout, facts = self._pack(entries)
        return self._context(self._upload(host), layout, facts)

    # ------------------------------------------------------------------ HIP graphs for decode steps
    def _launch_graph(self, prepared: "PreparedStep") -> Optional[torch.Tensor]:
        entries = prepared.entries
        B = len(entries)
        graph = self._graphs.get(prepared.graph_key)
        if graph is None:
            graph = self._capture(prepared.graph_key, prepared.host, prepared.layout, prepared.facts)
        else:
            if prepared.layout != graph.layout or prepared.facts["plans"] != graph.plan_facts:
                raise StepError("a step planner gave a decode step of the same batch and context bucket another "
                                "layout or other numbers than the captured graph has")
            self._send(prepared, into=graph.static_dev)
        graph.graph.replay()
        picked = prepared.facts["picked"]
        if not picked:
            return None
        if len(picked) == B:
            return graph.logits[:B]
        # some entries want nothing: their rows are left out by a gather fed from the packed buffer
        first = prepared.layout["picked"][0]
        return ops.gather_rows(graph.logits, graph.static_dev[first:first + len(picked)])

    def _capture(self, key, host: np.ndarray, layout, facts) -> "_DecodeGraph":
        static_dev = torch.empty(host.size, dtype=torch.int32, device=self.env.device)
        self._upload(host, into=static_dev)
        ctx, rows = self._context(static_dev, layout, facts)
        with torch.no_grad():
            # once eagerly on a side stream: loads the kernels and sizes the library's workspaces.  Keys and
            # values written twice are the same keys and values; state that a step moves on is put back.
            states = [c.state for c in self._views.values() if c.state is not None]
            saved = [t.clone() for t in states]
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                self._forward(static_dev, layout, ctx, rows)
                for t, was in zip(states, saved):
                    t.copy_(was)
            torch.cuda.current_stream().wait_stream(side)
            if self._graph_pool is None:
                self._graph_pool = torch.cuda.graph_pool_handle()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, pool=self._graph_pool):
                logits = self._forward(static_dev, layout, ctx, rows)
        graph = _DecodeGraph(g, static_dev, logits, dict(layout), dict(facts["plans"]))
        self._graphs[key] = graph
        return graph


@dataclass
class PreparedStep:
    """A step whose host work is done (see :meth:`ModelRunner.prepare`)."""
    entries: List[StepEntry]
    host: np.ndarray                  # the packed batch description
    layout: dict                      # field name -> (first, end) in it
    facts: dict
    graph_key: Optional[tuple]        # (batch bucket, context bucket) if the step replays a graph
    staged: Optional[torch.Tensor] = None   # the description already in pinned memory (see ModelRunner.stage)

    def unknown_tokens(self) -> List[tuple]:
        """(entry, index among the entry's tokens) of every token that still needs an id."""
        return [(b, j) for _, _, b, j in self.facts["unknown"]]

    def fill_token(self, k: int, token: int) -> None:
        """Give the k-th unknown token its id."""
        at = self.facts["unknown"][k][0]
        self.host[at] = token
        if self.staged is not None:
            self.staged[at] = token

    def feed_token(self, k: int, index: int) -> None:
        """The k-th unknown token is entry ``index`` of the runner's ``feed_source`` when the step runs."""
        at = self.facts["unknown"][k][1]
        self.host[at] = index
        if self.staged is not None:
            self.staged[at] = index

    def all_tokens_known(self) -> None:
        self.facts["unknown"] = []


@dataclass
class _DecodeGraph:
    graph: "torch.cuda.CUDAGraph"
    static_dev: torch.Tensor          # the packed batch description the captured kernels read
    logits: torch.Tensor              # float32 [batch bucket, vocab], rewritten by every replay
    layout: dict                      # where the captured kernels read each field
    plan_facts: dict                  # the planners' numbers the kernels were launched with

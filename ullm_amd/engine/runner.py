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
from ..kernels.ops import PREFILL_TILE as Q_TILE   # tokens of one request per prompt-portion attention tile
from ..models.model import Model
from ..parts import GroupView, LayerCache, PartEnv, StepContext
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
        for g, spec in enumerate(groups):
            k_shape = (num_pages[g], spec.num_kv_heads, page_size, spec.head_dim)
            v_shape = (num_pages[g], spec.num_kv_heads, spec.head_dim, page_size)   # transposed inside a page
            for key in spec.layers:
                # zeroed once so that no row ever holds a non-finite bit pattern before it is written
                views[key] = LayerCache(
                    group=g, k_pool=torch.zeros(k_shape, dtype=env.dtype, device=env.device),
                    v_pool=torch.zeros(v_shape, dtype=env.dtype, device=env.device))
        for key, need in states.items():
            # one row more than requests: the slot of a captured batch's padding entries
            views[key] = LayerCache(
                state=torch.zeros((max_requests + 1,) + tuple(need.shape), dtype=need.dtype, device=env.device))
        self._views = views
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
            for t in (c.k_pool, c.v_pool, c.state):
                if t is not None:
                    total += t.numel() * t.element_size()
        return total

    def _pack(self, entries: Sequence[StepEntry], pad_entries: int = 0, table_stride: Optional[int] = None,
              allow_unknown: bool = False):
        """Flatten the entries into one int32 host array.  Returns (host array, offsets, facts).
        ``pad_entries`` > len(entries) appends one-token entries that hold no pages (their cache
        writes are skipped and their outputs ignored), so that a batch fits a captured graph.
        With ``allow_unknown`` a token may be UNKNOWN_TOKEN (its id is filled in before the launch);
        ``facts["unknown"]`` lists such tokens as (index into the array, entry, index in the entry)."""
        P = self.page_size
        n_real = len(entries)
        lens = [len(e.tokens) for e in entries]
        if n_real == 0 or sum(lens) == 0:
            raise StepError("a step needs at least one token")
        n_pad = max(0, pad_entries - n_real)
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
        n_want = sum(len(e.want) for e in entries) + n_pad
        # attention work lists: tokens of one-token entries; tiles of <= Q_TILE tokens of longer entries
        dec_keys, tile_keys, max_dec_kv, t0 = [], [], 0, 0
        for e, n in zip(entries, lens):
            if n == 1:
                dec_keys.append((-e.cache.num_computed, t0))
                max_dec_kv = max(max_dec_kv, e.cache.num_computed + 1)
            else:
                for first in range(0, n, Q_TILE):
                    count = min(Q_TILE, n - first)
                    tile_keys.append((e.cache.num_computed + first + count, t0 + first, count))
            t0 += n
        tile_keys.sort()                                  # the attention kernel wants rising numbers of keys
        dec_keys.sort()                                   # longest contexts first: the short ones fill the tail
        dec_list = [t for _, t in dec_keys]
        tile_list = [x for _, first, count in tile_keys for x in (first, count)]
        dec_list.extend(range(t0, t0 + n_pad))
        ng = len(groups)
        sizes = [T, T, T, B + 1, B, B, n_want] + [B * s for s in strides] + [len(dec_list), len(tile_list), T]
        offs = np.concatenate(([0], np.cumsum(sizes)))
        host = np.zeros(int(offs[-1]), dtype=np.int32)
        ids, pos, ent = host[offs[0]:offs[1]], host[offs[1]:offs[2]], host[offs[2]:offs[3]]
        q_start, slot, start = host[offs[3]:offs[4]], host[offs[4]:offs[5]], host[offs[5]:offs[6]]
        rows = host[offs[6]:offs[7]]
        host[offs[9 + ng]:offs[10 + ng]] = -1             # per token: where the device takes its id from (-1: from ids)
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
                unknown.append((t, b, t - int(first_of[b])))
            tok[tok == UNKNOWN_TOKEN] = 0
        if int(tok.min()) < 0 or int(tok.max()) >= self.vocab_size:
            bad = next(rc for rc, e in zip(caches, entries) if min(e.tokens) < 0 or max(e.tokens) >= self.vocab_size)
            raise StepError(f"request {bad.request_id!r}: token id outside [0, {self.vocab_size})")
        ids[:n_tok] = tok
        slot[:n_real] = slots
        slot[n_real:] = self.padding_slot
        start[:n_real] = starts
        r = 0
        for b, e in enumerate(entries):
            for w in e.want:
                if not (0 <= w < lens[b]):
                    raise StepError(f"request {caches[b].request_id!r}: wanted place {w} outside its {lens[b]} tokens")
                rows[r] = q_start[b] + w
                r += 1
        max_kv = max(s0 + n for s0, n in zip(starts, lens))
        t = n_tok
        for b in range(n_real, B):                       # padding entries: token 0 at position 0, no pages
            ent[t] = b
            q_start[b] = t
            rows[r] = t
            t += 1
            r += 1
        q_start[B] = T
        for g, s in enumerate(strides):
            bt = host[offs[7 + g]:offs[8 + g]].reshape(B, s)
            bt[:n_real] = self.cache.table_rows(g, slots, s)
            bt[n_real:] = -1
        host[offs[7 + ng]:offs[8 + ng]] = dec_list
        host[offs[8 + ng]:offs[9 + ng]] = tile_list
        facts = dict(T=T, B=B, strides=strides, n_want=n_want, num_decode=len(dec_list), max_dec_kv=max_dec_kv,
                     num_tiles=len(tile_list) // 2, tile_keys_total=sum(k for k, _, _ in tile_keys),
                     tile_keys_max=tile_keys[-1][0] if tile_keys else 0, max_q=max(lens), max_kv=max_kv,
                     decode_only=all(n == 1 for n in lens), lens=lens + [1] * n_pad,
                     starts=starts + [0] * n_pad, slots=slots + [self.padding_slot] * n_pad, unknown=unknown)
        return host, offs, facts

    def _context(self, dev: torch.Tensor, offs, facts) -> tuple:
        """Views into the uploaded buffer as a StepContext, and the wanted rows."""
        groups = self.cache.groups
        ng = len(groups)
        B, T = facts["B"], facts["T"]
        view = lambda i: dev[int(offs[i]):int(offs[i + 1])]  # noqa: E731
        gviews = [GroupView(view(7 + g).view(B, facts["strides"][g]), facts["strides"][g], self.page_size,
                            groups[g].window) for g in range(ng)]
        ctx = StepContext(
            num_tokens=T, num_entries=B, token_ids=view(0), positions=view(1), token_entry=view(2),
            q_start=view(3), entry_slot=view(4), entry_start=view(5), groups=gviews,
            max_q_len=facts["max_q"], max_kv_len=facts["max_kv"], decode_only=facts["decode_only"],
            dtype=self.env.dtype,
            decode_tokens=view(7 + ng) if facts["num_decode"] else None, num_decode=facts["num_decode"],
            max_decode_kv=facts["max_dec_kv"], tiles=view(8 + ng).view(-1, 2) if facts["num_tiles"] else None,
            num_tiles=facts["num_tiles"], tile_keys_total=facts["tile_keys_total"],
            tile_keys_max=facts["tile_keys_max"], stacked_branches=self._stacked_branches,
            host={"lens": facts["lens"], "starts": facts["starts"], "slots": facts["slots"]})
        return ctx, (view(6) if facts["n_want"] else None)

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
            packed = [StepEntry(e.cache, e.tokens, [0]) for e in entries]
            host, offs, facts = self._pack(packed, pad_entries=b_pad, table_stride=self.max_table,
                                           allow_unknown=allow_unknown)
            return PreparedStep(entries, host, offs, facts, (b_pad, kv_bucket))
        host, offs, facts = self._pack(entries, allow_unknown=allow_unknown)
        return PreparedStep(entries, host, offs, facts, None)

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
        fresh = self.cache.take_fresh_slots()
        if fresh:
            for c in self._views.values():
                if c.state is not None:
                    c.state[torch.tensor(fresh, device=c.state.device)] = 0
        if prepared.graph_key is not None:
            logits = self._launch_graph(prepared)
        else:
            dev = self._send(prepared)
            self._feed(dev, prepared.offs)
            ctx, rows = self._context(dev, prepared.offs, prepared.facts)
            with torch.no_grad():
                logits = self.model.forward(ctx, self.caches, rows)
        for e in entries:
            self.cache.commit(e.cache, len(e.tokens))
        return logits

    def _feed(self, dev: torch.Tensor, offs) -> None:
        """Token ids that the step before has sampled and the host has not seen (see
        :meth:`PreparedStep.feed_token`) are taken from ``feed_source`` on the device."""
        if self.feed_source is not None:
            last = len(offs) - 1
            ops.feed_tokens(dev[int(offs[0]):int(offs[1])], dev[int(offs[last - 1]):int(offs[last])], self.feed_source)

    def build_context(self, entries: Sequence[StepEntry]):
        """Flatten the entries into device tensors (one host-to-device copy)."""
        host, offs, facts = self._pack(entries)
        return self._context(self._upload(host), offs, facts)

    # ------------------------------------------------------------------ HIP graphs for decode steps
    def _launch_graph(self, prepared: "PreparedStep") -> Optional[torch.Tensor]:
        entries = prepared.entries
        B = len(entries)
        graph = self._graphs.get(prepared.graph_key)
        if graph is None:
            graph = self._capture(prepared.graph_key, prepared.host, prepared.offs, prepared.facts)
        else:
            self._send(prepared, into=graph.static_dev)
        graph.graph.replay()
        wanted = [b for b, e in enumerate(entries) if len(e.want)]
        if not wanted:
            return None
        if len(wanted) == B:
            return graph.logits[:B]
        return graph.logits[torch.tensor(wanted, device=graph.logits.device)]

    def _capture(self, key, host: np.ndarray, offs, facts) -> "_DecodeGraph":
        b_pad, kv_bucket = key
        facts = dict(facts, max_dec_kv=kv_bucket, max_kv=kv_bucket)    # the kernels' split of the keys is fixed
        static_dev = torch.empty(host.size, dtype=torch.int32, device=self.env.device)
        self._upload(host, into=static_dev)
        ctx, rows = self._context(static_dev, offs, facts)
        with torch.no_grad():
            # once eagerly on a side stream: loads the kernels and sizes the library's workspaces.  Keys and
            # values written twice are the same keys and values; state that a step moves on is put back.
            states = [c.state for c in self._views.values() if c.state is not None]
            saved = [t.clone() for t in states]
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                self._feed(static_dev, offs)
                self.model.forward(ctx, self.caches, rows)
                for t, was in zip(states, saved):
                    t.copy_(was)
            torch.cuda.current_stream().wait_stream(side)
            if self._graph_pool is None:
                self._graph_pool = torch.cuda.graph_pool_handle()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, pool=self._graph_pool):
                self._feed(static_dev, offs)
                logits = self.model.forward(ctx, self.caches, rows)
        graph = _DecodeGraph(g, static_dev, logits)
        self._graphs[key] = graph
        return graph


@dataclass
class PreparedStep:
    """A step whose host work is done (see :meth:`ModelRunner.prepare`)."""
    entries: List[StepEntry]
    host: np.ndarray                  # the packed batch description
    offs: np.ndarray
    facts: dict
    graph_key: Optional[tuple]        # (batch bucket, context bucket) if the step replays a graph
    staged: Optional[torch.Tensor] = None   # the description already in pinned memory (see ModelRunner.stage)

    def unknown_tokens(self) -> List[tuple]:
        """(entry, index among the entry's tokens) of every token that still needs an id."""
        return [(b, j) for _, b, j in self.facts["unknown"]]

    def fill_token(self, k: int, token: int) -> None:
        """Give the k-th unknown token its id."""
        at = int(self.offs[0]) + self.facts["unknown"][k][0]
        self.host[at] = token
        if self.staged is not None:
            self.staged[at] = token

    def feed_token(self, k: int, index: int) -> None:
        """The k-th unknown token is entry ``index`` of the runner's ``feed_source`` when the step runs."""
        t = self.facts["unknown"][k][0]
        at = int(self.offs[len(self.offs) - 2]) + t
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

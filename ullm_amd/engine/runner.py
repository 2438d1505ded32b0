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
from ..models.model import Model
from ..parts import GroupView, LayerCache, PartEnv, StepContext


@dataclass
class StepEntry:
    """One request's next tokens.  ``want`` lists the places among these tokens whose logits are
    returned (it may be empty)."""
    cache: RequestCache
    tokens: Sequence[int]
    want: Sequence[int] = field(default_factory=list)


class StepError(RuntimeError):
    pass


Q_TILE = 16     # tokens of one request that the prompt-portion attention kernel handles per wave


class ModelRunner:
    def __init__(self, model: Model, env: PartEnv, page_size: int, num_pages, max_requests: int,
                 enable_prefix_cache: bool = False):
        if model.env is None:
            raise StepError("the model has no weights bound")
        self.model, self.env = model, env
        self.page_size = page_size
        self.max_requests = max_requests
        groups, cache_group, states = model.cache_layout()
        if isinstance(num_pages, int):
            num_pages = [num_pages] * len(groups)
        self.cache = CacheManager(groups, list(num_pages), page_size, max_requests,
                                  enable_prefix_cache=enable_prefix_cache and not states)
        self.max_table = -(-env.context_len // page_size)
        self.caches: Dict[int, LayerCache] = {}
        for g, spec in enumerate(groups):
            k_shape = (num_pages[g], spec.num_kv_heads, page_size, spec.head_dim)
            v_shape = (num_pages[g], spec.num_kv_heads, spec.head_dim, page_size)   # transposed inside a page
            for cache_id in spec.layers:
                # zeroed once so that no row ever holds a non-finite bit pattern before it is written
                self.caches[cache_id] = LayerCache(
                    group=g, k_pool=torch.zeros(k_shape, dtype=env.dtype, device=env.device),
                    v_pool=torch.zeros(v_shape, dtype=env.dtype, device=env.device))
        for cache_id, need in states.items():
            self.caches[cache_id] = LayerCache(
                state=torch.zeros((max_requests,) + tuple(need.shape), dtype=need.dtype, device=env.device))
        self._pin = env.device.type == "cuda"
        self._staging: List[Optional[torch.Tensor]] = [None, None]   # two host buffers, used in turn
        self._staging_done: List[Optional[torch.cuda.Event]] = [None, None]
        self._turn = 0
        self.vocab_size = model.plan.vocab_size

    # ------------------------------------------------------------------ helpers
    def cache_bytes(self) -> int:
        total = 0
        for c in self.caches.values():
            for t in (c.k_pool, c.v_pool, c.state):
                if t is not None:
                    total += t.numel() * t.element_size()
        return total

    def _upload(self, host: np.ndarray) -> torch.Tensor:
        """Copy the packed batch description to the device through one of two pinned buffers; a
        buffer is written again only after the copy that last read it has finished."""
        i = self._turn
        self._turn ^= 1
        if self._staging_done[i] is not None:
            self._staging_done[i].synchronize()
        if self._staging[i] is None or self._staging[i].numel() < host.size:
            self._staging[i] = torch.empty(max(host.size, 4096), dtype=torch.int32, pin_memory=self._pin)
        stage = self._staging[i][:host.size]
        stage.numpy()[:] = host
        dev = stage.to(self.env.device, non_blocking=True)
        if self._pin:
            ev = torch.cuda.Event()
            ev.record()
            self._staging_done[i] = ev
        elif dev.data_ptr() == stage.data_ptr():
            dev = dev.clone()
        return dev

    def build_context(self, entries: Sequence[StepEntry]):
        """Flatten the entries into device tensors (one host-to-device copy)."""
        P = self.page_size
        B = len(entries)
        lens = [len(e.tokens) for e in entries]
        T = sum(lens)
        if B == 0 or T == 0:
            raise StepError("a step needs at least one token")
        groups = self.cache.groups
        strides = []
        for g in range(len(groups)):
            strides.append(max(1, max(len(e.cache.tables[g]) for e in entries)))
        n_want = sum(len(e.want) for e in entries)
        # attention work lists: tokens of one-token entries; tiles of <= 16 tokens of longer entries
        dec_list, tile_list, max_dec_kv, t0 = [], [], 0, 0
        for e, n in zip(entries, lens):
            if n == 1:
                dec_list.append(t0)
                max_dec_kv = max(max_dec_kv, e.cache.num_computed + 1)
            else:
                for first in range(0, n, Q_TILE):
                    tile_list.extend((t0 + first, min(Q_TILE, n - first)))
            t0 += n
        # layout of the packed int32 buffer
        sizes = [T, T, T, B + 1, B, B, n_want] + [B * s for s in strides] + [len(dec_list), len(tile_list)]
        offs = np.concatenate(([0], np.cumsum(sizes)))
        host = np.empty(int(offs[-1]), dtype=np.int32)
        ids, pos, ent = host[offs[0]:offs[1]], host[offs[1]:offs[2]], host[offs[2]:offs[3]]
        q_start, slot, start = host[offs[3]:offs[4]], host[offs[4]:offs[5]], host[offs[5]:offs[6]]
        rows = host[offs[6]:offs[7]]
        t = 0
        r = 0
        max_kv = 0
        seen = set()
        for b, e in enumerate(entries):
            rc, n = e.cache, lens[b]
            if n < 1:
                raise StepError(f"request {rc.request_id!r}: an entry needs at least one token")
            if rc.released:
                raise StepError(f"request {rc.request_id!r} was released")
            if id(rc) in seen:
                raise StepError(f"request {rc.request_id!r} appears twice in one step")
            seen.add(id(rc))
            s0 = rc.num_computed
            if s0 + n > self.env.context_len:
                raise StepError(f"request {rc.request_id!r}: {s0 + n} tokens exceed context_len={self.env.context_len}")
            for g in range(len(groups)):
                if len(rc.tables[g]) * P < s0 + n:
                    raise StepError(f"request {rc.request_id!r}: no pages reserved for positions up to {s0 + n - 1}")
            tok = np.asarray(e.tokens, dtype=np.int64)
            if tok.min() < 0 or tok.max() >= self.vocab_size:
                raise StepError(f"request {rc.request_id!r}: token id outside [0, {self.vocab_size})")
            ids[t:t + n] = tok
            pos[t:t + n] = np.arange(s0, s0 + n)
            ent[t:t + n] = b
            q_start[b] = t
            slot[b] = rc.slot
            start[b] = s0
            for w in e.want:
                if not (0 <= w < n):
                    raise StepError(f"request {rc.request_id!r}: wanted place {w} outside its {n} tokens")
                rows[r] = t + w
                r += 1
            max_kv = max(max_kv, s0 + n)
            t += n
        q_start[B] = T
        for g, s in enumerate(strides):
            bt = host[offs[7 + g]:offs[8 + g]].reshape(B, s)
            bt.fill(-1)
            for b, e in enumerate(entries):
                tab = e.cache.tables[g]
                bt[b, :len(tab)] = tab
        ng = len(groups)
        host[offs[7 + ng]:offs[8 + ng]] = dec_list
        host[offs[8 + ng]:offs[9 + ng]] = tile_list
        dev = self._upload(host)
        view = lambda i: dev[int(offs[i]):int(offs[i + 1])]  # noqa: E731
        gviews = [GroupView(view(7 + g).view(B, strides[g]), strides[g], P, groups[g].window)
                  for g in range(len(groups))]
        ctx = StepContext(
            num_tokens=T, num_entries=B, token_ids=view(0), positions=view(1), token_entry=view(2),
            q_start=view(3), entry_slot=view(4), entry_start=view(5), groups=gviews,
            max_q_len=max(lens), max_kv_len=max_kv, decode_only=all(n == 1 for n in lens),
            dtype=self.env.dtype,
            decode_tokens=view(7 + ng) if (dec_list and len(dec_list) < T) else None, num_decode=len(dec_list),
            max_decode_kv=max_dec_kv, tiles=view(8 + ng).view(-1, 2) if tile_list else None,
            num_tiles=len(tile_list) // 2,
            host={"lens": lens, "starts": [e.cache.num_computed for e in entries],
                  "slots": [e.cache.slot for e in entries]})
        return ctx, (view(6) if n_want else None)

    # ------------------------------------------------------------------ the step
    def step(self, entries: Sequence[StepEntry]) -> Optional[torch.Tensor]:
        """Run the entries as one batch.  Pages for the new tokens must have been reserved.
        Returns float32 logits [number of wanted places, vocab] in the order of the entries and of
        their ``want`` lists, or None if nothing is wanted.  On return the requests' caches hold the
        new tokens (``num_computed`` has advanced)."""
        fresh = self.cache.take_fresh_slots()
        if fresh:
            for c in self.caches.values():
                if c.state is not None:
                    c.state[torch.tensor(fresh, device=c.state.device)] = 0
        ctx, rows = self.build_context(entries)
        with torch.no_grad():
            logits = self.model.forward(ctx, self.caches, rows)
        for e in entries:
            self.cache.commit(e.cache, len(e.tokens))
        return logits

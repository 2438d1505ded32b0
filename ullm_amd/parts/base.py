"""What every part of a layer has in common: declared weights, declared cache needs,
and a registry from (kind, name) to the class, so that a model is put together from a
plan that names its parts layer by layer.

Kinds: "mixer" (attention or anything else that mixes tokens), "ffn" (feed-forward),
"norm", "position" (position encoding) and "block" (how norm, mixer and feed-forward are
arranged around the residual stream).  No part knows which model it is in: sizes and
constants arrive as constructor parameters, tensor names as a prefix.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional, Tuple, Union

import torch


# --------------------------------------------------------------------------- weights

@dataclass(frozen=True)
class WeightDecl:
    """One tensor a part binds by its checkpoint name."""
    name: str
    shape: Tuple[int, ...]
    init: str = "normal"          # random mode: "normal" N(0,s) | "gain" 1+N(0,s)
    keep_fp32: bool = False       # held in 32-bit whatever the compute dtype (norm gains)
    alias_of: Optional[str] = None  # if absent from the checkpoint, bind this tensor instead
    # A tensor that is used only as rows ``row_offset ..`` of a larger matrix (q | k | v, gate | up)
    # names that matrix here.  The loader allocates the matrix once, copies every such tensor into its
    # rows, and hands ``bind`` the matrix under the name ``merged_into`` (not the pieces); a checkpoint
    # that already holds the whole matrix under that name is taken as it is.
    merged_into: Optional[str] = None
    row_offset: int = 0


# --------------------------------------------------------------------------- cache needs

@dataclass(frozen=True)
class CacheRows:
    """One pool of a paged cache: per token and head a row of ``dim`` values.  The pool is
    [pages, heads, page_size, dim], or with ``transposed`` [pages, heads, dim, page_size] (a page's tokens
    side by side for every dim)."""
    name: str
    heads: int
    dim: int
    transposed: bool = False
    dtype: Optional[torch.dtype] = None      # None: the compute dtype


@dataclass(frozen=True)
class KVNeed:
    """A mixer that keeps rows per token in pages.  By default one key row and one value row per token
    and kv head (pools "k" [pages, kv_heads, page_size, head_dim] and "v", transposed inside the page,
    [pages, kv_heads, head_dim, page_size]: the layout the attention kernels read).  A mixer that keeps
    something else per token (one latent row, keys only, rows in another dtype) names its pools in
    ``rows``; it then gets exactly those, as ``cache.pools[name]``, and nothing else."""
    num_kv_heads: int
    head_dim: int
    window: int = 0               # keys a query looks back over, itself included; 0 = all
    rows: Tuple[CacheRows, ...] = ()

    def pools(self) -> Tuple[CacheRows, ...]:
        if self.rows:
            return self.rows
        return (CacheRows("k", self.num_kv_heads, self.head_dim),
                CacheRows("v", self.num_kv_heads, self.head_dim, transposed=True))


@dataclass(frozen=True)
class StateNeed:
    """A mixer that keeps state of fixed size per request (zeroed at admission).

    ``graph_safe``: the mixer's step for single new tokens (``ctx.decode_only``) takes everything from
    device tensors (``ctx.entry_slot``, not the host lists), so it may be captured into a HIP graph and
    replayed with other requests in the same places.  The state tensor has one row more than there are
    requests; the padding entries of a captured batch carry that row's index as their slot, so whatever a
    step does to their state lands where no request looks.  One mixer that does not say so keeps the
    whole model on eager steps."""
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32
    graph_safe: bool = False


CacheNeed = Union[KVNeed, StateNeed, None]


def cache_needs_of(block) -> Tuple[Union[KVNeed, StateNeed], ...]:
    """What a block keeps between steps as a tuple: ``Block.cache_need()`` may return nothing, one
    need, or a list of needs (a block with keys and values and fixed-size state, or with two shapes
    of keys)."""
    need = block.cache_need()
    if need is None:
        return ()
    if isinstance(need, (KVNeed, StateNeed)):
        return (need,)
    needs = tuple(need)
    for n in needs:
        if not isinstance(n, (KVNeed, StateNeed)):
            raise TypeError(f"{type(block).__name__}.cache_need() returned {n!r}: not a KVNeed or StateNeed")
    return needs


# --------------------------------------------------------------------------- step context

@dataclass
class GroupView:
    """Block tables of the batch entries for one cache group (device tensors)."""
    block_table: torch.Tensor     # int32 [B, stride]; entry = page id, -1 where none is held
    stride: int
    page_size: int
    window: int


@dataclass
class LayerCache:
    """What a mixer sees of the cache: its layer's pools or its layer's state rows.

    A block that declares several needs gets one view per need, in the order declared, as ``parts``
    and hands each of its mixers the one that is its own (``cache.parts[i]``); the outer view's own
    fields then show the first need of each kind, so a block with one need never looks at ``parts``."""
    group: int = -1                        # index into StepContext.groups for KV mixers
    k_pool: Optional[torch.Tensor] = None  # pools["k"]: [num_pages, kv_heads, page_size, head_dim]
    v_pool: Optional[torch.Tensor] = None  # pools["v"]: [num_pages, kv_heads, head_dim, page_size]
    state: Optional[torch.Tensor] = None   # [num_slots, *StateNeed.shape]
    owner: bool = True                     # False: reads another layer's cache, writes nothing
    parts: List["LayerCache"] = field(default_factory=list)
    pools: Dict[str, torch.Tensor] = field(default_factory=dict)   # every pool the need declared, by name

    @staticmethod
    def of_pools(group: int, pools: Dict[str, torch.Tensor]) -> "LayerCache":
        return LayerCache(group=group, k_pool=pools.get("k"), v_pool=pools.get("v"), pools=dict(pools))

    @staticmethod
    def of_parts(parts: List["LayerCache"]) -> "LayerCache":
        """The view of a block from the views of its needs."""
        if len(parts) == 1:
            return parts[0]
        kv = next((p for p in parts if p.pools), None)
        st = next((p for p in parts if p.state is not None), None)
        return LayerCache(group=kv.group if kv else -1, k_pool=kv.k_pool if kv else None,
                          v_pool=kv.v_pool if kv else None, state=st.state if st else None, parts=list(parts),
                          pools=dict(kv.pools) if kv else {})

    def reader(self) -> "LayerCache":
        """The same cache for a layer that only reads it."""
        return LayerCache(self.group, self.k_pool, self.v_pool, self.state, owner=False,
                          parts=[p.reader() for p in self.parts], pools=self.pools)


@dataclass(frozen=True)
class StepShape:
    """What a step planner is told about a batch (host numbers only)."""
    lens: Tuple[int, ...]         # new tokens of each entry, in batch order
    starts: Tuple[int, ...]       # tokens each entry's request holds in the cache before the step
    pad_entries: int = 0          # one-token entries appended behind them for a captured graph: position 0, no pages
    kv_bucket: Optional[int] = None   # the step replays a captured graph: launch shapes must be those of this context length


@dataclass
class StepPlan:
    """A kernel family's own view of a step: work lists (int32 arrays; they travel to the device inside
    the step's one packed buffer and come back as tensors) and host numbers (grid sizes, counts).

    A part names the planners its kernels need in ``Part.step_planners`` ({name: function of a
    :class:`StepShape`}); the step function runs each once per step and the part finds the result as
    ``ctx.plans[name]``.  For a step that replays a captured graph (``shape.kv_bucket`` is set) the arrays'
    sizes may depend only on the number of entries including padding, and the numbers only on that and
    the bucket: the captured kernels read the arrays at fixed places and were launched with those numbers."""
    arrays: Dict[str, object] = field(default_factory=dict)   # host: numpy int32 arrays; in a StepContext: device tensors
    facts: Dict[str, int] = field(default_factory=dict)


@dataclass
class StepContext:
    """Device-side description of one batch: T tokens of B entries, flattened."""
    num_tokens: int
    num_entries: int
    token_ids: torch.Tensor       # int32 [T]
    positions: torch.Tensor       # int32 [T] absolute position of each token in its request
    token_entry: torch.Tensor     # int32 [T] batch entry each token belongs to
    q_start: torch.Tensor         # int32 [B+1] first token of each entry
    entry_slot: torch.Tensor      # int32 [B] request slot of each entry (state rows)
    entry_start: torch.Tensor     # int32 [B] position of the entry's first token
    groups: List[GroupView]
    max_q_len: int                # host copies, for grids
    max_kv_len: int
    decode_only: bool             # every entry brings exactly one token
    dtype: torch.dtype = torch.bfloat16          # compute dtype of activations
    host: dict = field(default_factory=dict)   # host-side copies for parts that want them
    # what the planners named by the model's parts made of this step (Part.step_planners), by name
    plans: Dict[str, StepPlan] = field(default_factory=dict)
    # every norm of the model takes a stack [S, T, hidden] of float32 partial sums as its branch and
    # adds them up (Norm.adds_stacks): a mixer or feed-forward may then return such a stack
    stacked_branches: bool = False


# --------------------------------------------------------------------------- parts

@dataclass(frozen=True)
class PartEnv:
    """Where and how a model is built: handed to every part with its tensors."""
    device: torch.device
    dtype: torch.dtype            # compute dtype: torch.bfloat16 or torch.float32
    context_len: int              # most positions any request reaches
    # tensors that parts of many layers would otherwise each build for themselves (position tables):
    # built once per key and shared, see ``shared``
    _shared: Dict[tuple, torch.Tensor] = field(default_factory=dict, compare=False, repr=False)

    def shared(self, key: tuple, build: Callable[[], torch.Tensor]) -> torch.Tensor:
        """The tensor of this key, built by ``build()`` the first time it is asked for.  The key must
        name everything the tensor depends on (kind, sizes, constants, rows)."""
        t = self._shared.get(key)
        if t is None:
            t = self._shared[key] = build()
        return t


class Part:
    """Base of every part.  ``weights()`` declares tensors; ``bind`` receives them.

    ``graph_safe``: the part's work in a step of single new tokens can be captured into a HIP graph: it
    queues the same kernels whatever the tokens are and never waits for the device (no sizes that
    depend on values, as a routed feed-forward that gathers each expert's rows has).  One part that
    says no keeps the whole model on eager steps."""
    kind = ""
    graph_safe = True
    # {name: function(StepShape) -> StepPlan}: per-step work lists this part's kernels want (see StepPlan)
    step_planners: Dict[str, Callable] = {}

    def weights(self) -> List[WeightDecl]:
        return []

    def bind(self, tensors: Dict[str, torch.Tensor], env: PartEnv) -> None:
        """Called once with {declared name: device tensor in its final dtype}."""

    def children(self) -> List["Part"]:
        return []


class Mixer(Part):
    """Token mixer: ``forward(x [T, hidden], ctx, cache) -> [T, hidden]`` in the compute dtype.

    A mixer may also offer ``forward_fused(x, residual, ctx, cache)``: add mixer(x) into the 32-bit
    residual in place, with the add folded into its last kernel.  It is called only when
    ``fusable(residual, ctx)`` says so.  With ``folds_norm`` its ``forward_fused`` also takes a
    :class:`PendingNorm` for x: the norm before it, left to the mixer's first projection.
    With ``hands_norm_ahead`` its ``forward_fused`` also takes ``then=``, the norm that will be applied to the
    stream next (or None), and may return that norm as a :class:`PendingNorm` that its last kernel prepared
    (the stream times the gain, the rows' sums of squares); it returns None where it prepared nothing."""
    kind = "mixer"
    folds_norm = False
    hands_norm_ahead = False

    def cache_need(self) -> CacheNeed:
        return None

    def forward(self, x: torch.Tensor, ctx: StepContext, cache: LayerCache) -> torch.Tensor:
        raise NotImplementedError

    def fusable(self, residual: torch.Tensor, ctx: StepContext) -> bool:
        return False

    def forward_fused(self, x, residual, ctx: StepContext, cache: LayerCache) -> None:
        raise NotImplementedError


class FeedForward(Part):
    """``forward(x [T, hidden], ctx) -> [T, hidden]``; keeps nothing between steps.
    ``fusable``, ``forward_fused(x, residual, ctx)``, ``folds_norm`` and ``hands_norm_ahead`` as for mixers."""
    kind = "ffn"
    folds_norm = False
    hands_norm_ahead = False

    def forward(self, x: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        raise NotImplementedError

    def fusable(self, residual: torch.Tensor, ctx: StepContext) -> bool:
        return False

    def forward_fused(self, x, residual, ctx: StepContext) -> None:
        raise NotImplementedError


class PendingNorm:
    """A norm of the residual stream that has not been computed: what a consumer needs to fold it
    into its first projection (``stream`` float32 [T, hidden], ``gain`` float32 [hidden], ``eps``;
    the scale is rsqrt(mean of squares + eps)), and ``apply()`` for a consumer that cannot after all.
    Where the product that wrote the stream last prepared the norm, also ``scaled`` (stream * gain in the
    compute dtype) and ``squares`` (float32 [T, parts]: a row's sum of squares in parts): the consumer then
    multiplies ``scaled`` and scales row t of its results by rsqrt(squares[t].sum() / hidden + eps)."""

    def __init__(self, norm: "Norm", stream: torch.Tensor, gain: torch.Tensor, eps: float, out_dtype: torch.dtype,
                 scaled: Optional[torch.Tensor] = None, squares: Optional[torch.Tensor] = None):
        self.norm, self.stream, self.gain, self.eps, self.out_dtype = norm, stream, gain, eps, out_dtype
        self.scaled, self.squares = scaled, squares

    def apply(self) -> torch.Tensor:
        return self.norm.add_norm(None, self.stream, out_dtype=self.out_dtype)


class Norm(Part):
    """``add_norm(branch, residual, rows) -> normed``: adds the branch output (if any) into
    the 32-bit residual stream, then normalises the sum; ``rows`` selects output rows.
    ``adds_stacks``: the branch may also be a stack [S, T, hidden] of float32 partial sums, which
    the norm adds in order.
    ``pending(residual, out_dtype)``: a :class:`PendingNorm` of a stream with nothing left to add, for
    a consumer with ``folds_norm``, or None if this norm has no such form; with ``scaled`` and ``squares``
    where a product prepared them.  ``ahead_gain()``: the float32 gain [hidden] such a product multiplies
    the stream by, or None if this norm is not a gain times rsqrt(mean of squares + eps)."""
    kind = "norm"
    adds_stacks = False

    def pending(self, residual: torch.Tensor, out_dtype: torch.dtype, scaled: Optional[torch.Tensor] = None,
                squares: Optional[torch.Tensor] = None) -> Optional["PendingNorm"]:
        return None

    def ahead_gain(self) -> Optional[torch.Tensor]:
        return None

    def add_norm(self, branch: Optional[torch.Tensor], residual: torch.Tensor,
                 rows: Optional[torch.Tensor] = None, out_dtype: torch.dtype = None) -> torch.Tensor:
        raise NotImplementedError


class PositionEncoding(Part):
    """Describes how query and key vectors are marked with their position.
    ``kernel_args()`` -> (table tensor or None, rotary_dim, style) for the fused
    norm/rotate/cache-write kernel; style 0 = none, 1 = half-split pairs, 2 = adjacent pairs."""
    kind = "position"

    def kernel_args(self):
        return None, 0, 0


class Block(Part):
    """Arrangement of norm, mixer and feed-forward around the residual stream.

    ``forward(residual, pending, ctx, cache) -> (residual, pending)`` where ``residual`` is the
    32-bit stream [T, hidden] and ``pending`` a branch output not yet added to it.

    A block with ``hands_norm_ahead`` takes ``next_norm=`` in ``forward``: the norm that the next block of the
    run order applies to the stream first (that block's ``entry_norm()``), or None.  It may then return a
    :class:`PendingNorm` of that norm as its pending branch (nothing is left to add; the norm is half done),
    which is only ever given to the block whose ``entry_norm()`` it is."""
    kind = "block"
    hands_norm_ahead = False

    def entry_norm(self) -> Optional["Norm"]:
        return None

    def cache_need(self):
        """Nothing, one need (``KVNeed`` / ``StateNeed``) or a list of needs; with a list the block
        gets ``cache.parts`` in the same order."""
        return None

    def forward(self, residual, pending, ctx: StepContext, cache: LayerCache):
        raise NotImplementedError


# --------------------------------------------------------------------------- registry

_PARTS: Dict[str, Dict[str, Callable]] = {k: {} for k in ("mixer", "ffn", "norm", "position", "block")}


def register_part(kind: str, name: str):
    """Class decorator: make ``build_part(kind, name, ...)`` construct this class."""
    if kind not in _PARTS:
        raise KeyError(f"unknown part kind {kind!r}; kinds are {sorted(_PARTS)}")

    def deco(cls):
        _PARTS[kind][name] = cls
        return cls
    return deco


def build_part(kind: str, name: str, **params) -> Part:
    try:
        cls = _PARTS[kind][name]
    except KeyError:
        raise KeyError(f"no {kind} part named {name!r}; registered: {sorted(_PARTS.get(kind, {}))}") from None
    return cls(**params)


def registered_parts(kind: str) -> List[str]:
    return sorted(_PARTS[kind])


def walk(part: Part):
    """The part and every part below it."""
    yield part
    for c in part.children():
        yield from walk(c)

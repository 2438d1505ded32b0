"""Python faces of the HIP kernels: each checks operand shapes, dtypes and contiguity on the host,
then launches on torch's current stream through the family's ``extern "C"`` entry point.
A non-zero return of a launcher raises ``KernelError``; nothing falls back to another path.
"""
from __future__ import annotations

import ctypes
import logging
from typing import Optional

import torch

from . import build, dispatch

F32, BF16 = 0, 1
logger = logging.getLogger("ullm_amd")


class KernelError(RuntimeError):
    pass


_ERR_NAMES = {-1: "unsupported dtype combination", -2: "operand shape outside what the kernel takes",
              -3: "unsupported argument combination", -4: "partial results exceed the fixed scratch array"}


def _check(rc: int, what: str) -> None:
    if rc != 0:
        reason = _ERR_NAMES.get(rc, f"HIP error {rc}")
        raise KernelError(f"{what}: {reason}")


def _dt(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return F32
    if t.dtype == torch.bfloat16:
        return BF16
    raise KernelError(f"dtype {t.dtype} is not float32 or bfloat16")


def _stream() -> ctypes.c_void_p:
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _p(t: Optional[torch.Tensor]) -> ctypes.c_void_p:
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelError(msg)


def _i32(t: torch.Tensor, name: str, n: Optional[int] = None) -> None:
    _need(t.dtype == torch.int32 and t.is_contiguous(), f"{name} must be contiguous int32")
    if n is not None:
        _need(t.numel() >= n, f"{name} holds {t.numel()} entries, {n} needed")


_c_int, _c_float = ctypes.c_int, ctypes.c_float


def _check_pools(k_pool, v_pool, nkv: int, page_size: int, hd: int, dtype) -> None:
    """Keys are [pages, nkv, page_size, hd]; values are kept transposed inside a page: [pages, nkv, hd, page_size]."""
    _need(k_pool is not None and k_pool.dim() == 4 and tuple(k_pool.shape[1:]) == (nkv, page_size, hd)
          and k_pool.is_contiguous() and k_pool.dtype == dtype,
          f"k_pool must be contiguous [pages, {nkv}, {page_size}, {hd}] of {dtype}")
    _need(v_pool is not None and v_pool.dim() == 4 and tuple(v_pool.shape[1:]) == (nkv, hd, page_size)
          and v_pool.is_contiguous() and v_pool.dtype == dtype and v_pool.shape[0] == k_pool.shape[0],
          f"v_pool must be contiguous [pages, {nkv}, {hd}, {page_size}] of {dtype}")


# ---------------------------------------------------------------------------------- elementwise

def embedding(ids: torch.Tensor, table: torch.Tensor, out: Optional[torch.Tensor] = None, scale: float = 1.0) -> torch.Tensor:
    """float32 [T, H] rows of ``table`` [V, H] at ``ids`` [T] (int32), times ``scale``."""
    T = ids.numel()
    V, H = table.shape
    _i32(ids, "ids")
    _need(table.is_contiguous(), "embedding table must be contiguous")
    if out is None:
        out = torch.empty((T, H), dtype=torch.float32, device=table.device)
    _need(out.dtype == torch.float32 and out.is_contiguous() and out.shape == (T, H), "bad embedding output")
    lib = build.load("elementwise")
    _check(lib.ullm_embedding(_p(ids), _p(table), _p(out), _c_int(T), _c_int(H), _c_int(V),
                              _c_int(_dt(table)), _c_float(scale), _stream()), "embedding")
    return out


def softcap_(x: torch.Tensor, cap: float) -> torch.Tensor:
    """x = cap * tanh(x / cap) in place, float32 [rows, cols]."""
    _need(x.dtype == torch.float32 and x.dim() == 2 and x.stride(1) == 1 and cap > 0, "softcap takes float32 [rows, cols] and a cap > 0")
    _check(build.load("elementwise").ullm_softcap(_p(x), _c_int(x.shape[0]), _c_int(x.shape[1]), _c_int(x.stride(0)),
                                                  _c_float(cap), _stream()), "softcap")
    return x


def feed_tokens(ids: torch.Tensor, feed: torch.Tensor, source: torch.Tensor) -> None:
    """ids[t] = source[feed[t]] wherever feed[t] >= 0 (all int32): token ids that the step before has
    sampled and the host has not yet seen are taken from that step's output on the device."""
    n = ids.numel()
    _i32(ids, "ids")
    _i32(feed, "feed", n)
    _i32(source, "source")
    _check(build.load("elementwise").ullm_feed_tokens(_p(ids), _p(feed), _p(source), _c_int(n),
                                                      _c_int(source.numel()), _stream()), "feed_tokens")


def zero_fresh_rows(state: torch.Tensor, entry_slot: torch.Tensor, entry_start: torch.Tensor, n_entries: int) -> None:
    """state[entry_slot[b]] = 0 for every entry b < n_entries with entry_start[b] == 0: the per-request state
    rows (``state`` contiguous [slots, anything]) of requests that step from their first token.  Takes
    everything from device tensors, so it can be part of a captured step."""
    _need(state.is_contiguous() and state.dim() >= 1, "state must be contiguous [slots, ...]")
    _i32(entry_slot, "entry_slot", n_entries)
    _i32(entry_start, "entry_start", n_entries)
    rows = state.shape[0]
    row_bytes = (state.numel() // max(1, rows)) * state.element_size()
    _check(build.load("elementwise").ullm_zero_fresh_rows(_p(state), ctypes.c_longlong(row_bytes), _c_int(rows),
                                                         _p(entry_slot), _p(entry_start), _c_int(n_entries), _stream()),
           "zero_fresh_rows")


def gather_rows(src: torch.Tensor, index: torch.Tensor) -> torch.Tensor:
    """src[index] for float32 ``src`` [n, cols] and int32 ``index`` on the device: no index travels from the
    host and nothing waits for the device."""
    _need(src.dtype == torch.float32 and src.dim() == 2 and src.stride(1) == 1, "gather_rows takes float32 [n, cols]")
    _i32(index, "index")
    n, cols = index.numel(), src.shape[1]
    out = torch.empty((n, cols), dtype=torch.float32, device=src.device)
    _check(build.load("elementwise").ullm_gather_rows(_p(src), ctypes.c_longlong(src.stride(0)), _c_int(src.shape[0]),
                                                     _p(index), _p(out), _c_int(n), _c_int(cols), _stream()), "gather_rows")
    return out


def stream_read(src: torch.Tensor, blocks: int = 0) -> torch.Tensor:
    """Read ``src`` (contiguous, a multiple of 16 bytes) once with a kernel that does nothing else; returns the
    words the blocks stored (their xor of what they read).  For measuring what a read-only kernel reaches."""
    nbytes = src.numel() * src.element_size()
    _need(src.is_contiguous() and nbytes % 16 == 0 and src.data_ptr() % 16 == 0, "stream_read takes contiguous, 16-byte aligned memory")
    n_blocks = blocks if blocks > 0 else 8 * compute_units(src.device)
    sink = torch.empty(n_blocks * 4, dtype=torch.int32, device=src.device)
    _check(build.load("elementwise").ullm_stream_read(_p(src), ctypes.c_longlong(nbytes), _p(sink), _c_int(n_blocks), _stream()),
           "stream_read")
    return sink


def add_rmsnorm(branch: Optional[torch.Tensor], residual: torch.Tensor, gain: torch.Tensor, eps: float,
                out_dtype: torch.dtype, rows: Optional[torch.Tensor] = None,
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """residual (float32 [T, H], updated in place unless ``rows``) += branch; returns the RMS-normed
    sum times ``gain`` (float32 [H]) in ``out_dtype``.  With ``rows`` (int32 [n]) only those rows are
    produced and the residual stays untouched.  ``branch`` may be a stack [S, T, H] of partial sums
    (see :func:`gemm_partial_sums`): they are added in order."""
    T, H = residual.shape
    _need(residual.dtype == torch.float32 and residual.is_contiguous(), "residual must be contiguous float32")
    _need(gain.dtype == torch.float32 and gain.numel() == H and gain.is_contiguous(), "gain must be float32 [H]")
    n_branch, branch_stride = 1, 0
    if branch is not None:
        _need(branch.shape[-2:] == (T, H) and branch.dim() in (2, 3) and branch.is_contiguous(),
              "branch must be contiguous [T, H] or a stack [S, T, H]")
        if branch.dim() == 3:
            n_branch, branch_stride = branch.shape[0], T * H
    n = T
    if rows is not None:
        _i32(rows, "rows")
        n = rows.numel()
    if out is None:
        out = torch.empty((n, H), dtype=out_dtype, device=residual.device)
    _need(out.shape == (n, H) and out.is_contiguous() and out.dtype == out_dtype, "bad norm output")
    lib = build.load("elementwise")
    bdt = _dt(branch) if branch is not None else _dt(out)
    _check(lib.ullm_add_rmsnorm(_p(branch), _p(residual), _p(gain), _c_float(eps), _p(out), _p(rows),
                                _c_int(n), _c_int(H), _c_int(bdt), _c_int(_dt(out)),
                                _c_int(0 if rows is not None else 1), _c_int(n_branch),
                                ctypes.c_longlong(branch_stride), _stream()), "add_rmsnorm")
    return out


def residual_add(branch: torch.Tensor, residual: torch.Tensor) -> None:
    """residual (float32, contiguous) += branch (same shape, contiguous)."""
    _need(residual.dtype == torch.float32 and residual.is_contiguous() and branch.is_contiguous()
          and branch.shape == residual.shape, "residual_add takes contiguous tensors of one shape")
    lib = build.load("elementwise")
    _check(lib.ullm_residual_add(_p(branch), _p(residual), ctypes.c_longlong(residual.numel()), _c_int(_dt(branch)),
                                 _stream()), "residual_add")


def add_bias(y: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """y [T, N] += bias (float32 [N]) in place, the sum taken in 32-bit; returns y."""
    T, N = y.shape
    _need(y.stride(1) == 1, "y must have unit stride along its rows")
    _need(bias.dtype == torch.float32 and bias.numel() == N and bias.is_contiguous(), "bias must be float32 [N]")
    _check(build.load("elementwise").ullm_add_bias(_p(y), _p(bias), _c_int(T), _c_int(N), ctypes.c_longlong(y.stride(0)),
                                                   _c_int(_dt(y)), _stream()), "add_bias")
    return y


def silu_mul(gate_up: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """silu(gate_up[:, :I]) * gate_up[:, I:] for a contiguous [T, 2I] input."""
    T, two_i = gate_up.shape
    _need(two_i % 2 == 0 and gate_up.is_contiguous(), "gate_up must be contiguous [T, 2I]")
    inter = two_i // 2
    if out is None:
        out = torch.empty((T, inter), dtype=gate_up.dtype, device=gate_up.device)
    _need(out.shape == (T, inter) and out.is_contiguous() and out.dtype == gate_up.dtype, "bad silu_mul output")
    lib = build.load("elementwise")
    _check(lib.ullm_silu_mul(_p(gate_up), _p(out), _c_int(T), _c_int(inter), _c_int(_dt(gate_up)), _stream()),
           "silu_mul")
    return out


def sum_stacks(stacks: torch.Tensor, bias: Optional[torch.Tensor] = None,
               out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """The sum over the first dimension of float32 ``stacks`` [S, M, N] (what :func:`gemm_partial_sums` leaves), added
    in order, plus ``bias`` [N], as [M, N] of ``out_dtype``."""
    _need(stacks.dtype == torch.float32 and stacks.dim() == 3 and stacks.is_contiguous() and stacks.shape[2] % 4 == 0,
          "stacks must be contiguous float32 [S, M, N] with N a multiple of 4")
    S, M, N = stacks.shape
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.numel() == N and bias.is_contiguous(), "bias must be float32 [N]")
    out = torch.empty((M, N), dtype=out_dtype, device=stacks.device)
    lib = build.load("elementwise")
    _check(lib.ullm_sum_stacks(_p(stacks), _c_int(S), _p(bias), _p(out), _c_int(M), _c_int(N), _c_int(_dt(out)), _stream()),
           "sum_stacks")
    return out


def qk_norm_rope_write(qkv: torch.Tensor, q_out: torch.Tensor, q_gain: Optional[torch.Tensor],
                       k_gain: Optional[torch.Tensor], eps: float, cos_sin: Optional[torch.Tensor],
                       rotary_dim: int, style: int, positions: torch.Tensor, token_entry: torch.Tensor,
                       block_table: torch.Tensor, k_pool: Optional[torch.Tensor], v_pool: Optional[torch.Tensor],
                       page_size: int, nq: int, nkv: int, hd: int, write_kv: bool) -> None:
    """Per-head norm and rotation of q (to ``q_out`` [T, nq*hd]) and k, and the cache write of k and v.
    ``qkv`` is [T, (nq + 2 nkv) * hd]; key pool [pages, nkv, page_size, hd], value pool
    [pages, nkv, hd, page_size]; ``block_table`` is
    int32 [B, stride] with one row per batch entry."""
    T = qkv.shape[0]
    _need(qkv.dim() == 2 and qkv.shape[1] == (nq + 2 * nkv) * hd and qkv.stride(1) == 1, "bad qkv shape")
    _need(q_out.shape == (T, nq * hd) and q_out.is_contiguous() and q_out.dtype == qkv.dtype, "bad q_out")
    _need(hd <= 512, f"head_dim {hd} exceeds 512")
    _i32(positions, "positions", T)
    _i32(token_entry, "token_entry", T)
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.stride(1) == 1,
          "block_table must be int32 [B, stride]")
    for g, nm in ((q_gain, "q_gain"), (k_gain, "k_gain")):
        if g is not None:
            _need(g.dtype == torch.float32 and g.numel() == hd and g.is_contiguous(), f"{nm} must be float32 [hd]")
    table_rows = 0
    if style != 0 and rotary_dim > 0:
        _need(cos_sin is not None and cos_sin.dtype == torch.float32 and cos_sin.dim() == 2
              and cos_sin.shape[1] == rotary_dim and cos_sin.is_contiguous(),
              "cos_sin must be float32 [positions, rotary_dim]")
        table_rows = cos_sin.shape[0]
    if write_kv:
        _check_pools(k_pool, v_pool, nkv, page_size, hd, qkv.dtype)
    lib = build.load("elementwise")
    _check(lib.ullm_qk_norm_rope_write(
        _p(qkv), _c_int(qkv.stride(0)), _p(q_out), _c_int(q_out.stride(0)), _p(q_gain), _p(k_gain),
        _c_float(eps), _p(cos_sin), _c_int(table_rows), _c_int(rotary_dim), _c_int(style), _p(positions),
        _p(token_entry), _p(block_table), _c_int(block_table.stride(0)), _p(k_pool), _p(v_pool),
        _c_int(page_size), _c_int(T), _c_int(nq), _c_int(nkv), _c_int(hd), _c_int(1 if write_kv else 0),
        _c_int(_dt(qkv)), _stream()), "qk_norm_rope_write")


# ---------------------------------------------------------------------------------- attention

def paged_attention_generic(q: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                            positions: torch.Tensor, token_entry: torch.Tensor, block_table: torch.Tensor,
                            page_size: int, nq: int, nkv: int, hd: int, scale: float, window: int,
                            out: Optional[torch.Tensor] = None) -> torch.Tensor:
    T = q.shape[0]
    _need(q.shape == (T, nq * hd) and q.stride(1) == 1, "q must be [T, nq*hd]")
    _need(hd <= 512 and nq % nkv == 0, "head_dim > 512 or heads not a multiple of kv heads")
    _check_pools(k_pool, v_pool, nkv, page_size, hd, q.dtype)
    _i32(positions, "positions", T)
    _i32(token_entry, "token_entry", T)
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.stride(1) == 1,
          "block_table must be int32 [B, stride]")
    if out is None:
        out = torch.empty((T, nq * hd), dtype=q.dtype, device=q.device)
    _need(out.shape == (T, nq * hd) and out.is_contiguous() and out.dtype == q.dtype, "bad attention output")
    lib = build.load("attention_generic")
    _check(lib.ullm_paged_attention_generic(
        _p(q), _c_int(q.stride(0)), _p(out), _c_int(out.stride(0)), _p(k_pool), _p(v_pool), _p(positions),
        _p(token_entry), _p(block_table), _c_int(block_table.stride(0)), _c_int(page_size), _c_int(T),
        _c_int(nq), _c_int(nkv), _c_int(hd), _c_float(scale), _c_int(window), _c_int(_dt(q)), _stream()),
        "paged_attention_generic")
    return out


# ---------------------------------------------------------------------------------- matrix products

def gemm_simple(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None,
                out_dtype: Optional[torch.dtype] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """a [M, K] times w [N, K] transposed (+ bias float32 [N]); 32-bit multiply-add in fixed K order."""
    M, K = a.shape
    N, K2 = w.shape
    _need(K == K2, f"inner sizes differ: a is [{M}, {K}], w is [{N}, {K2}]")
    _need(a.stride(1) == 1 and w.stride(1) == 1, "a and w must have unit stride along K")
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype or a.dtype, device=a.device)
    _need(out.shape == (M, N) and out.stride(1) == 1, "bad gemm output")
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.numel() == N and bias.is_contiguous(), "bias must be float32 [N]")
    lib = build.load("gemm_simple")
    _check(lib.ullm_gemm_simple(_p(a), _c_int(a.stride(0)), _p(w), _c_int(w.stride(0)), _p(bias), _p(out),
                                _c_int(out.stride(0)), _c_int(M), _c_int(N), _c_int(K), _c_int(_dt(a)),
                                _c_int(_dt(w)), _c_int(_dt(out)), _stream()), "gemm_simple")
    return out


def _skinny_ok(M: int, K: int, x: torch.Tensor, w: torch.Tensor) -> bool:
    return (w.dtype == torch.bfloat16 and 1 <= M <= 64 and K % 8 == 0 and K >= 8 and x.stride(1) == 1
            and w.stride(1) == 1 and x.stride(0) % 8 == 0 and w.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0
            and w.data_ptr() % 16 == 0)


def gemm_skinny_supports(a: torch.Tensor, w: torch.Tensor) -> bool:
    return a.dtype == torch.bfloat16 and _skinny_ok(a.shape[0], a.shape[1], a, w)


def _gemm_skinny(x, w, bias, c, M, N, K, epi, c_dtype, nt=0, waves=0, gain=None, eps=0.0, rows=0,
                 ahead=None, squares=None) -> None:
    """``ahead``: (next gain, next x, next squares) that an adding product leaves for the norm after it;
    ``squares``: the [parts, M] sums such a product left, which scale this product's rows."""
    lib = build.load("gemm_skinny")
    next_gain, next_x, next_sq = ahead if ahead is not None else (None, None, None)
    _check(lib.ullm_gemm_skinny(_p(x), _c_int(x.stride(0)), _p(w), _c_int(w.stride(0)), _p(bias),
                                _p(c), _c_int(c.stride(0)), _c_int(M), _c_int(N), _c_int(K),
                                _c_int(epi), _c_int(c_dtype), _c_int(nt), _c_int(waves), _p(gain),
                                ctypes.c_float(eps), _c_int(rows), _p(next_gain), _p(next_x),
                                _c_int(next_x.stride(0) if next_x is not None else 0), _p(next_sq), _p(squares),
                                _c_int(squares.shape[1] if squares is not None else 0), _stream()),
           "gemm_skinny")


def _check_squares(squares: Optional[torch.Tensor], M: int) -> None:
    if squares is not None:
        _need(M <= 16 and squares.dtype == torch.float32 and squares.dim() == 2 and squares.shape[0] == M
              and squares.shape[1] >= 4 and squares.shape[1] % 4 == 0 and squares.is_contiguous()
              and squares.data_ptr() % 16 == 0, f"row squares must be float32 [{M} <= 16, a multiple of 4]")


def gemm_skinny(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None,
                out_dtype: Optional[torch.dtype] = None, out: Optional[torch.Tensor] = None,
                nt: int = 0, waves: int = 0, rows: int = 0, squares: Optional[torch.Tensor] = None,
                eps: float = 0.0) -> torch.Tensor:
    """a [M <= 64, K] times w [N, K] transposed, bfloat16 operands streamed once through the matrix
    cores, 32-bit accumulation; output bfloat16 or float32.  With ``squares`` (float32 [M <= 16, parts], see
    :func:`gemm_skinny_add`) row m of the product is scaled by rsqrt(sum of squares[m] / K + eps) before
    the bias: a is then a stream times a norm's gain and the result the product of the normed stream."""
    M, K = a.shape
    N, K2 = w.shape
    _need(K == K2, f"inner sizes differ: a is [{M}, {K}], w is [{N}, {K2}]")
    _need(gemm_skinny_supports(a, w), "gemm_skinny takes bfloat16, M <= 64, K a multiple of 8, 16-byte aligned rows")
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype or a.dtype, device=a.device)
    _need(out.shape == (M, N) and out.stride(1) == 1, "bad gemm output")
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.numel() == N and bias.is_contiguous(), "bias must be float32 [N]")
    _check_squares(squares, M)
    _gemm_skinny(a, w, bias, out, M, N, K, 0, _dt(out), nt, waves, eps=float(eps), rows=rows, squares=squares)
    return out


def gemm_skinny_add(a: torch.Tensor, w: torch.Tensor, residual: torch.Tensor, nt: int = 0, waves: int = 0,
                    rows: int = 0, next_gain: Optional[torch.Tensor] = None):
    """residual (float32 [M, N]) += a (bfloat16 [M, K]) times w transposed.
    With ``next_gain`` (float32 [N], the gain of the RMS norm that is applied to the residual next) the kernel
    also leaves what that norm needs and returns it: (scaled, squares) with scaled = residual * next_gain in
    bfloat16 [M, N] and squares float32 [M, parts], every block's sum of the squares of its columns of a row
    (zeros behind them up to a multiple of four).
    The norm of row m is scaled[m] * rsqrt(squares[m].sum() / N + eps), which a product after it applies
    to its own results (``squares=`` of :func:`gemm_skinny`, :func:`gemm_skinny_silu`, :func:`gemm_rows`)."""
    M = a.shape[0]
    N, K = w.shape
    _need(a.dtype == torch.bfloat16 and a.shape[1] == K and _skinny_ok(M, K, a, w),
          "gemm_skinny_add takes bfloat16 activations [M <= 64, K]")
    _need(residual.dtype == torch.float32 and residual.shape == (M, N) and residual.stride(1) == 1
          and residual.stride(0) % 4 == 0 and residual.data_ptr() % 16 == 0, "residual must be float32 [M, N]")
    if next_gain is None:
        _gemm_skinny(a, w, None, residual, M, N, K, 1, F32, nt, waves, rows=rows)
        return None
    _need(next_gain.dtype == torch.float32 and next_gain.numel() == N and next_gain.is_contiguous()
          and next_gain.data_ptr() % 16 == 0 and N % 4 == 0, "the next norm's gain must be float32 [N], N a multiple of 4")
    blocks = int(build.load("gemm_skinny").ullm_gemm_skinny_blocks(
        _c_int(M), _c_int(N), _c_int(K), _c_int(a.stride(0)), _c_int(w.stride(0)), _c_int(1), _c_int(nt), _c_int(waves),
        _c_int(rows)))
    _check(min(blocks, 0), "gemm_skinny_blocks")
    scaled = torch.empty((M, N), dtype=torch.bfloat16, device=a.device)
    squares = torch.empty((M, -(-blocks // 4) * 4), dtype=torch.float32, device=a.device)
    _gemm_skinny(a, w, None, residual, M, N, K, 1, F32, nt, waves, rows=rows, ahead=(next_gain, scaled, squares))
    return scaled, squares


def gemm_skinny_silu(a: torch.Tensor, w_gate_up: torch.Tensor, nt: int = 0, waves: int = 0, rows: int = 0,
                     squares: Optional[torch.Tensor] = None, eps: float = 0.0) -> torch.Tensor:
    """silu(a g^T) * (a u^T) as bfloat16 [M, I] for a (bfloat16 [M, K]) and the stacked weights
    g | u (bfloat16 [2 I, K]); the activation is applied to the 32-bit sums (with ``squares``: to the sums
    scaled as in :func:`gemm_skinny`)."""
    M, K = a.shape
    two_i, K2 = w_gate_up.shape
    _need(K == K2 and two_i % 2 == 0, f"gate|up weights must be [2 I, {K}]")
    _need(a.dtype == torch.bfloat16 and _skinny_ok(M, K, a, w_gate_up), "gemm_skinny_silu takes bfloat16 [M <= 64, K]")
    out = torch.empty((M, two_i // 2), dtype=torch.bfloat16, device=a.device)
    _check_squares(squares, M)
    _gemm_skinny(a, w_gate_up, None, out, M, two_i // 2, K, 2, BF16, nt, waves, eps=float(eps), rows=rows, squares=squares)
    return out


NORMED_MAX_ROWS = 16


def gemm_skinny_normed_supports(stream: torch.Tensor, gain: torch.Tensor, w: torch.Tensor) -> bool:
    M, K = stream.shape
    return (stream.dtype == torch.float32 and gain.dtype == torch.float32 and w.dtype == torch.bfloat16
            and M <= NORMED_MAX_ROWS and gain.numel() == K and gain.is_contiguous() and gain.data_ptr() % 16 == 0
            and _skinny_ok(M, K, stream, w))


def gemm_skinny_normed(stream: torch.Tensor, gain: torch.Tensor, eps: float, w: torch.Tensor,
                       bias: Optional[torch.Tensor] = None, out_dtype: torch.dtype = torch.bfloat16,
                       silu: bool = False, nt: int = 0, waves: int = 0, rows: int = 0) -> torch.Tensor:
    """rmsnorm(stream) times w transposed for the float32 residual stream [M <= 16, K], the norm
    (gain float32 [K], eps) folded into the product: the kernel rounds stream * gain to bfloat16 for
    the matrix cores, sums the squares of the rows it reads anyway and scales the 32-bit sums by
    rsqrt(mean + eps).  With silu, w is gate | up [2 I, K] and the result silu(gate) * up [M, I]."""
    M, K = stream.shape
    N, K2 = w.shape
    _need(K == K2, f"inner sizes differ: the stream is [{M}, {K}], w is [{N}, {K2}]")
    _need(gemm_skinny_normed_supports(stream, gain, w),
          "gemm_skinny_normed takes a float32 stream [M <= 16, K], a float32 gain [K] and bfloat16 weights")
    if silu:
        _need(N % 2 == 0 and bias is None and out_dtype == torch.bfloat16, "gate|up weights must be [2 I, K], no bias")
        N //= 2
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.numel() == N and bias.is_contiguous(), "bias must be float32 [N]")
    out = torch.empty((M, N), dtype=out_dtype, device=stream.device)
    _gemm_skinny(stream, w, bias, out, M, N, K, 2 if silu else 0, _dt(out), nt, waves, gain, float(eps), rows)
    return out


PARTIAL_SUMS_MAX_ROWS = 256


def gemm_partial_sums_supports(a: torch.Tensor, w: torch.Tensor) -> bool:
    M, K = a.shape
    return (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and a.stride(1) == 1 and w.stride(1) == 1
            and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0 and w.shape[1] == K
            and bool(build.load("gemm_mid").ullm_gemm_partial_sums_supports(
                _c_int(M), _c_int(w.shape[0]), _c_int(K), _c_int(a.stride(0)), _c_int(w.stride(0)))))


def gemm_partial_sums(a: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """a (bfloat16 [M <= 256, K]) times w (bfloat16 [N, K]) transposed as a stack [S, M, N] of float32
    partial sums over S slices of K; the product is their sum.  S depends on the matrix alone.  For
    17 to 256 rows of the projections that end in the residual stream: the add + norm kernel adds the
    stack (:func:`add_rmsnorm`), so the slices cost no kernel of their own."""
    M, K = a.shape
    N = w.shape[0]
    _need(gemm_partial_sums_supports(a, w), "gemm_partial_sums takes bfloat16, M <= 256, K a multiple of 8, N of 4")
    lib = build.load("gemm_mid")
    slices = int(lib.ullm_gemm_partial_sums_slices(_c_int(N), _c_int(K)))
    out = torch.empty((slices, M, N), dtype=torch.float32, device=a.device)
    _check(lib.ullm_gemm_partial_sums(_p(a), _c_int(a.stride(0)), _p(w), _c_int(w.stride(0)), _p(out), _c_int(M),
                                      _c_int(N), _c_int(K), _stream()), "gemm_partial_sums")
    return out


ROWS_MAX_ROWS = 128       # most rows the kernel takes (which matrices it is chosen for: dispatch.limits)


def gemm_rows_supports(a: torch.Tensor, w: torch.Tensor, silu: bool = False) -> bool:
    M, K = a.shape
    n_out = w.shape[0] // 2 if silu else w.shape[0]
    return (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and a.stride(1) == 1 and w.stride(1) == 1
            and w.shape[1] == K and (not silu or w.shape[0] % 2 == 0) and a.data_ptr() % 16 == 0
            and w.data_ptr() % 16 == 0 and n_out % 4 == 0
            and bool(build.load("gemm_rows").ullm_gemm_rows_supports(
                _c_int(M), _c_int(n_out), _c_int(K), _c_int(a.stride(0)), _c_int(w.stride(0)), _c_int(n_out),
                _c_int(1 if silu else 0))))


def gemm_rows(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None, silu: bool = False,
              squares: Optional[torch.Tensor] = None, eps: float = 0.0) -> torch.Tensor:
    """a (bfloat16 [M <= 128, K]) times w (bfloat16 [N, K]) transposed (+ bias float32 [N]) as bfloat16 [M, N];
    with ``silu``, w is gate | up [2 I, K] and the result silu(gate) * up [M, I] on the 32-bit sums.  The
    matrix is cut into one block per compute unit and every wave keeps several stages of its rows of w in
    flight: for the row counts between the few-rows kernel and the library.  ``squares``, ``eps``: as in
    :func:`gemm_skinny`."""
    M, K = a.shape
    _need(gemm_rows_supports(a, w, silu), "gemm_rows takes bfloat16, M <= 128, K a multiple of 64, N a multiple of 4")
    n_out = w.shape[0] // 2 if silu else w.shape[0]
    if bias is not None:
        _need(not silu and bias.dtype == torch.float32 and bias.numel() == n_out and bias.is_contiguous(),
              "bias must be float32 [N] (and there is none with silu)")
    _check_squares(squares, M)
    out = torch.empty((M, n_out), dtype=torch.bfloat16, device=a.device)
    _check(build.load("gemm_rows").ullm_gemm_rows(_p(a), _c_int(a.stride(0)), _p(w), _c_int(w.stride(0)), _p(bias), _p(out),
                                                  _c_int(n_out), _c_int(M), _c_int(n_out), _c_int(K),
                                                  _c_int(1 if silu else 0), _p(squares),
                                                  _c_int(squares.shape[1] if squares is not None else 0),
                                                  ctypes.c_float(float(eps)), _stream()), "gemm_rows")
    return out


# torch.mm(..., out_dtype=float32) stores the 32-bit accumulator of a bfloat16 product; older torch lacks it
_MM_TAKES_OUT_DTYPE = "out_dtype" in (torch.mm.__doc__ or "")


def gemm_bf16(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None,
              out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """bfloat16 operands, 32-bit accumulation.  Few rows go to the weight-streaming kernels (up to how many
    for this matrix: :func:`dispatch.limits`), some more, where that was measured to be ahead, to the partial-sums
    kernel and a kernel that adds its stacks; many rows go through the library product (as the reference's
    linears do, ullm/layers/linear.py:165), which for 32-bit output (logits) stores the accumulator unrounded."""
    out_dtype = out_dtype or a.dtype
    M = a.shape[0]
    library = a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and a.is_cuda
    lim = dispatch.limits(w.shape[0], w.shape[1])
    few = lim.f32_skinny if out_dtype == torch.float32 else lim.skinny
    if M <= few and gemm_skinny_supports(a, w):
        return gemm_skinny(a, w, bias, out_dtype=out_dtype)
    if out_dtype == torch.bfloat16 and M <= min(lim.rows, ROWS_MAX_ROWS) and gemm_rows_supports(a, w):
        return gemm_rows(a, w, bias)
    if (out_dtype == torch.bfloat16 and 0 < lim.sums_from <= M <= lim.sums_to and w.shape[0] % 4 == 0
            and gemm_partial_sums_supports(a, w)):
        return sum_stacks(gemm_partial_sums(a, w), bias)
    if library and out_dtype == torch.float32 and a.is_contiguous() and w.is_contiguous() and _MM_TAKES_OUT_DTYPE:
        y = torch.mm(a, w.t(), out_dtype=torch.float32)
        return y if bias is None else add_bias(y, bias)
    if library and out_dtype == torch.bfloat16:
        y = torch.nn.functional.linear(a, w)
        return y if bias is None else add_bias(y, bias)
    if out_dtype == torch.float32 and M <= 64 and gemm_skinny_supports(a, w):
        return gemm_skinny(a, w, bias, out_dtype=out_dtype)
    return gemm_simple(a, w, bias, out_dtype=out_dtype)


def attention_mfma_supports(dtype: torch.dtype, hd: int, page_size: int, nq: int, nkv: int) -> bool:
    """True if the matrix-core attention kernels take this shape (bfloat16, head_dim in
    {32, 64, 96, 128, 256}, page size a multiple of 16)."""
    if dtype != torch.bfloat16:
        return False
    return bool(build.load("attention_mfma").ullm_attention_mfma_supports(
        _c_int(hd), _c_int(page_size), _c_int(nq), _c_int(nkv)))


_units_of_device = {}


def compute_units(device=None) -> int:
    """Compute units of the device the kernels run on (256 on an MI355X)."""
    index = torch.cuda.current_device() if device is None else torch.device(device).index or 0
    n = _units_of_device.get(index)
    if n is None:
        n = _units_of_device[index] = int(torch.cuda.get_device_properties(index).multi_processor_count)
    return n


def decode_split(n_items: int, nkv: int, groups: int, max_kv: int, hd: int = 128, window: int = 0, units: int = 256):
    """(waves, num_splits) of the decode attention launch.  A wave walks its keys one 32-key tile after
    the other, each a round trip to memory, so few (token, kv head) pairs with many keys are cut over
    several blocks, up to one block per compute unit (more would run in a second round), and a second
    small kernel adds the blocks' partial results; that kernel costs about as much as walking eight more
    tiles, so short contexts are not cut.  Mostly a block is a single wave (several are resident on a
    SIMD, they start and end independently and one's start overlaps the others' streaming, and their number
    need not be a multiple of the compute units); four waves a block where few pairs have very many keys.
    With a window a token reads at most the window's keys (and up to 31 before them, to the tile's edge),
    however long its context is.  ``units``: the device's compute units, four SIMDs each."""
    pairs = max(1, n_items * nkv * groups)
    simds = 4 * units
    if pairs >= simds:
        return 1, 1
    if window > 0:
        max_kv = min(max_kv, window + 31)
    tiles = -(-max_kv // 32)
    if pairs > units:
        # single waves, two to four to a SIMD, so that the launch has no rounds of whole blocks (four-wave blocks,
        # one to a compute unit, take 49 us at 264 pairs against 30 us at 256); up to 2.25 pairs a unit cut in three
        # where that still gives at most one wave per SIMD and compute unit, else in two
        return 1, (max(2, min(3, simds // pairs)) if pairs <= units * 9 // 4 and tiles > 16 else 1)
    if pairs == units:
        return (4 if tiles > 16 else 1), 1
    # up to 16 blocks a pair; up to 32 where very few pairs have very many keys (one request at 4 096 keys and
    # more: 134 MB of cache at 32 768 keys in 34 us against 49 us with 16; three or four requests at 32 000 keys:
    # 70 and 89 us against 89 and 93 us; two requests are better off with 16 blocks of four waves)
    most = 32 if ((pairs * 128 <= simds and tiles >= 128) or (16 < pairs <= simds // 32 and tiles >= 512)) else 16
    splits = min(most, max(1, 2 * units // pairs), tiles)
    if tiles > 8 * splits:
        splits = min(most, max(1, simds // pairs), tiles)
    waves = 4 if (tiles > 4 * splits and pairs * splits * 4 <= simds) else 1
    return waves, splits


def attention_decode_mfma(q, out, k_pool, v_pool, token_list: Optional[torch.Tensor], n_items: int,
                          positions, token_entry, block_table, page_size: int, nq: int, nkv: int, hd: int,
                          scale: float, window: int, max_kv: int, splits: int = 0, waves: int = 0) -> None:
    """One query token per item (``token_list`` int32 [n_items] names the tokens, None = tokens
    0..n_items-1) against its request's cache; with ``splits`` > 1 the keys go to several blocks whose
    partial results a second small kernel adds up."""
    _check_pools(k_pool, v_pool, nkv, page_size, hd, torch.bfloat16)
    _need(q.dtype == torch.bfloat16 and q.stride(1) == 1 and q.shape[1] == nq * hd, "q must be bfloat16 [T, nq*hd]")
    _need(out.dtype == torch.bfloat16 and out.stride(1) == 1 and out.shape == q.shape, "bad attention output")
    _i32(positions, "positions")
    _i32(token_entry, "token_entry")
    if token_list is not None:
        _i32(token_list, "token_list", n_items)
    else:
        _need(n_items <= q.shape[0], "more items than tokens")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.stride(1) == 1,
          "block_table must be int32 [B, stride]")
    _need(-(-max_kv // page_size) <= block_table.shape[1], "block table narrower than the longest context")
    groups = -(-(nq // nkv) // 16)
    auto_waves, auto_splits = decode_split(n_items, nkv, groups, max_kv, hd, window, compute_units(q.device))
    waves = waves or auto_waves
    if hd == 256 and waves == 8:
        waves = 4
    splits = splits or auto_splits
    lib = build.load("attention_mfma")
    ws = None
    if splits > 1:
        ws = torch.empty(n_items * nq * splits * (hd + 4), dtype=torch.float32, device=q.device)
    _check(lib.ullm_attention_decode(
        _p(q), _c_int(q.stride(0)), _p(out), _c_int(out.stride(0)), _p(k_pool), _p(v_pool), _p(token_list),
        _c_int(n_items), _p(positions), _p(token_entry), _p(block_table), _c_int(block_table.stride(0)),
        _c_int(page_size), _c_int(nq), _c_int(nkv), _c_int(hd), _c_float(scale), _c_int(window),
        _c_int(splits), _c_int(waves), _p(ws), _stream()), "attention_decode")


def attention_decode_fused_supports(dtype: torch.dtype, hd: int, page_size: int, nq: int, nkv: int,
                                    rotary_dim: int, style: int) -> bool:
    """Whether the decode kernel can also do the step's per-head norm, rotation and cache write."""
    if dtype != torch.bfloat16:
        return False
    lib = build.load("attention_mfma")
    return bool(lib.ullm_attention_decode_fused_supports(_c_int(hd), _c_int(page_size), _c_int(nq), _c_int(nkv),
                                                         _c_int(rotary_dim), _c_int(style)))


def attention_decode_fused(qkv, out, q_gain: Optional[torch.Tensor], k_gain: Optional[torch.Tensor], eps: float,
                           cos_sin: Optional[torch.Tensor], rotary_dim: int, style: int, k_pool, v_pool,
                           token_list: Optional[torch.Tensor], n_items: int, positions, token_entry, block_table,
                           page_size: int, nq: int, nkv: int, hd: int, scale: float, window: int, max_kv: int,
                           write_kv: bool, splits: int = 0, waves: int = 0) -> None:
    """``attention_decode_mfma`` for a step in which every item is its request's newest token, with what
    ``qk_norm_rope_write`` does folded in: ``qkv`` [T, (nq + 2 nkv) * hd] is the fused projection as the
    matrix product left it; the kernel norms and rotates q and k itself and writes k and v to the cache."""
    _check_pools(k_pool, v_pool, nkv, page_size, hd, torch.bfloat16)
    _need(qkv.dtype == torch.bfloat16 and qkv.dim() == 2 and qkv.stride(1) == 1 and qkv.shape[1] == (nq + 2 * nkv) * hd,
          "qkv must be bfloat16 [T, (nq + 2 nkv) * hd]")
    _need(out.dtype == torch.bfloat16 and out.stride(1) == 1 and out.shape == (qkv.shape[0], nq * hd), "bad attention output")
    _i32(positions, "positions")
    _i32(token_entry, "token_entry")
    if token_list is not None:
        _i32(token_list, "token_list", n_items)
    else:
        _need(n_items <= qkv.shape[0], "more items than tokens")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.stride(1) == 1,
          "block_table must be int32 [B, stride]")
    _need(-(-max_kv // page_size) <= block_table.shape[1], "block table narrower than the longest context")
    for gn, nm in ((q_gain, "q_gain"), (k_gain, "k_gain")):
        if gn is not None:
            _need(gn.dtype == torch.float32 and gn.numel() == hd and gn.is_contiguous(), f"{nm} must be float32 [hd]")
    table_rows = 0
    if style != 0 and rotary_dim > 0:
        _need(cos_sin is not None and cos_sin.dtype == torch.float32 and cos_sin.dim() == 2
              and cos_sin.shape[1] == rotary_dim and cos_sin.is_contiguous(),
              "cos_sin must be float32 [positions, rotary_dim]")
        table_rows = cos_sin.shape[0]
    groups = -(-(nq // nkv) // 16)
    auto_waves, auto_splits = decode_split(n_items, nkv, groups, max_kv, hd, window, compute_units(qkv.device))
    waves = waves or auto_waves
    if hd == 256 and waves == 8:
        waves = 4
    splits = splits or auto_splits
    lib = build.load("attention_mfma")
    ws = None
    if splits > 1:
        ws = torch.empty(n_items * nq * splits * (hd + 4), dtype=torch.float32, device=qkv.device)
    _check(lib.ullm_attention_decode_fused(
        _p(qkv), _c_int(qkv.stride(0)), _p(out), _c_int(out.stride(0)), _p(k_pool), _p(v_pool), _p(token_list),
        _c_int(n_items), _p(positions), _p(token_entry), _p(block_table), _c_int(block_table.stride(0)),
        _c_int(page_size), _c_int(nq), _c_int(nkv), _c_int(hd), _c_float(scale), _c_int(window),
        _c_int(splits), _c_int(waves), _p(ws), _p(q_gain), _p(k_gain), _c_float(eps), _p(cos_sin),
        _c_int(table_rows), _c_int(rotary_dim), _c_int(style), _c_int(1 if write_kv else 0), _stream()),
        "attention_decode_fused")


PREFILL_TILE = 32      # tokens of one request per prompt tile (two groups of 16 columns for every wave of a block)


def attention_prefill_mfma(q, out, k_pool, v_pool, tiles: torch.Tensor, n_tiles: int, positions, token_entry,
                           block_table, page_size: int, nq: int, nkv: int, hd: int, scale: float,
                           window: int, halves: int = 0, keys_total: int = 0, keys_max: int = 0) -> None:
    """Tiles (first token, count <= PREFILL_TILE) of consecutive tokens of one request each, every
    token against the keys up to its own position.  ``halves``: 2 = two halves of a block share a
    tile's keys, 1 = one block takes them all, 0 = chosen from ``keys_total`` (the sum over the tiles of
    the keys each sees) and ``keys_max`` (the most any tile sees), or from the number of tiles if
    these are 0.  Every choice computes the same function."""
    _check_pools(k_pool, v_pool, nkv, page_size, hd, torch.bfloat16)
    _need(q.dtype == torch.bfloat16 and q.stride(1) == 1 and q.shape[1] == nq * hd, "q must be bfloat16 [T, nq*hd]")
    _need(out.dtype == torch.bfloat16 and out.stride(1) == 1 and out.shape == q.shape, "bad attention output")
    _need(tiles.dtype == torch.int32 and tiles.is_contiguous() and tiles.numel() >= 2 * n_tiles, "tiles must be int32 [n, 2]")
    _i32(positions, "positions")
    _i32(token_entry, "token_entry")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.stride(1) == 1,
          "block_table must be int32 [B, stride]")
    lib = build.load("attention_mfma")
    _check(lib.ullm_attention_prefill(
        _p(q), _c_int(q.stride(0)), _p(out), _c_int(out.stride(0)), _p(k_pool), _p(v_pool), _p(tiles),
        _c_int(n_tiles), _p(positions), _p(token_entry), _p(block_table), _c_int(block_table.stride(0)),
        _c_int(page_size), _c_int(nq), _c_int(nkv), _c_int(hd), _c_float(scale), _c_int(window),
        _c_int(halves), ctypes.c_longlong(int(keys_total)), _c_int(keys_max), _stream()),
        "attention_prefill")


_warned_general_attention = set()


def _warn_general_attention(hd: int, page_size: int) -> None:
    """Said once per shape: bfloat16 attention that the matrix-core kernels do not take runs on the general
    kernel (one block per token and head), which is right but many times slower."""
    if (hd, page_size) in _warned_general_attention:
        return
    _warned_general_attention.add((hd, page_size))
    why = []
    if hd not in (32, 64, 96, 128, 256):
        why.append(f"head_dim {hd} is not one of 32, 64, 96, 128, 256")
    if page_size % 16:
        why.append(f"page size {page_size} is not a multiple of 16")
    logger.warning("bfloat16 attention runs on the general kernel, not on the matrix cores (%s): expect it to be "
                   "many times slower", "; ".join(why) or "shape not supported")


def paged_attention(q: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor, ctx, group, nq: int,
                    nkv: int, hd: int, scale: float, window: int, plan=None) -> torch.Tensor:
    """Attention of the batch's queries over their requests' cached keys and values (the new
    tokens' rows included).  bfloat16 shapes the matrix-core kernels take go there (one launch for
    the one-token entries, one for the tiles of longer entries, both listed in ``plan``: arrays
    ``decode_tokens`` and ``tiles``, numbers ``num_decode``, ``max_decode_kv``, ``num_tiles``,
    ``tile_keys_total``, ``tile_keys_max``); everything else, and float32 always, takes the general
    kernel.  Every choice computes the same function."""
    if not attention_mfma_supports(q.dtype, hd, group.page_size, nq, nkv):
        if q.dtype == torch.bfloat16:
            _warn_general_attention(hd, group.page_size)
        return paged_attention_generic(q, k_pool, v_pool, ctx.positions, ctx.token_entry, group.block_table,
                                       group.page_size, nq, nkv, hd, scale, window)
    _need(plan is not None, "the matrix-core attention kernels need the step's work lists (a step plan)")
    out = torch.empty((q.shape[0], nq * hd), dtype=q.dtype, device=q.device)
    n = plan.facts
    if n["num_decode"]:
        attention_decode_mfma(q, out, k_pool, v_pool, plan.arrays["decode_tokens"], n["num_decode"], ctx.positions,
                              ctx.token_entry, group.block_table, group.page_size, nq, nkv, hd, scale, window,
                              n["max_decode_kv"])
    if n["num_tiles"]:
        attention_prefill_mfma(q, out, k_pool, v_pool, plan.arrays["tiles"], n["num_tiles"], ctx.positions,
                               ctx.token_entry, group.block_table, group.page_size, nq, nkv, hd, scale, window,
                               keys_total=n["tile_keys_total"], keys_max=n["tile_keys_max"])
    return out


# ---------------------------------------------------------------------------------- sampling

SAMPLE_PARTS_TOP_K = 64     # the largest top-k that the sampling kernels serve from parts of a row (PART_K_MAX)


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
           min_p: torch.Tensor, seed_lo: torch.Tensor, seed_hi: torch.Tensor, position: torch.Tensor,
           out: Optional[torch.Tensor] = None, parts: bool = True) -> torch.Tensor:
    """One token id per row of float32 ``logits`` [n, V].  Per-row parameters: temperature (0 =
    greedy), top_k (<= 0 = all), top_p, min_p (float32), seed halves and position (int32).  ``parts``: a first
    kernel cuts the rows into parts over many blocks where the settings allow (False: one block per row does
    everything)."""
    n, V = logits.shape
    _need(logits.dtype == torch.float32 and logits.stride(1) == 1, "logits must be float32 with unit stride")
    for t, nm, dt in ((temperature, "temperature", torch.float32), (top_k, "top_k", torch.int32),
                      (top_p, "top_p", torch.float32), (min_p, "min_p", torch.float32),
                      (seed_lo, "seed_lo", torch.int32), (seed_hi, "seed_hi", torch.int32),
                      (position, "position", torch.int32)):
        _need(t.dtype == dt and t.numel() >= n and t.is_contiguous(), f"{nm} must be contiguous {dt} [n]")
    if out is None:
        out = torch.empty((n,), dtype=torch.int32, device=logits.device)
    _need(out.dtype == torch.int32 and out.numel() >= n and out.is_contiguous(), "bad sample output")
    lib = build.load("sampling")
    lib.ullm_sample_workspace.restype = ctypes.c_longlong
    need = int(lib.ullm_sample_workspace(_c_int(n), _c_int(V), _c_int(logits.stride(0)))) if parts else 0
    ws = torch.empty(need, dtype=torch.float32, device=logits.device) if need > 0 else None
    _check(lib.ullm_sample(_p(logits), _c_int(n), _c_int(V), _c_int(logits.stride(0)), _p(temperature), _p(top_k),
                           _p(top_p), _p(min_p), _p(seed_lo), _p(seed_hi), _p(position), _p(out), _p(ws), _stream()),
           "sample")
    return out

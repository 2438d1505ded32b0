"""Times single kernels at given shapes: ``python -m ullm_amd.kernels.microbench <what> [options]``.

Every measurement records its calls as nodes of one HIP graph (so that a call costs what it costs
inside a decode graph, without the host's launch time) and rotates over several copies of the large
operands (weights, cache pages), enough of them that no call finds its data in the 256 MB memory-side
cache: the figures are those of a cold read from HBM, as in a model whose weights exceed that cache.

  decode-attention   one token per request over its cache: every (splits, waves) shape of the launch
  prefill-attention  prompt tiles of one request
  projection         a [rows, K] x [N, K]^T product by each kernel that can take it, and the library
  tune               the same for one matrix in the roles it has in a model; writes the row limits up to which
                     each kernel is ahead into the table that ullm_amd.kernels.dispatch reads
  sampling           the sampling kernels on rows of logits, per setting, with and without the kernel that cuts rows
                     into parts
"""
from __future__ import annotations

import argparse
from typing import Callable, List

import torch

from . import dispatch, ops

DEV = "cuda:0"


def graph_time(calls: List[Callable[[], None]], replays: int = 5) -> float:
    """Mean microseconds per call of ``calls`` when they run as one HIP graph.  A short list is repeated until
    the graph holds at least 24 calls, so that the launch of the graph itself is a small share of every call."""
    calls = list(calls) * max(1, -(-24 // max(1, len(calls))))
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for f in calls:
            f()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for f in calls:
            f()
    g.replay()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(replays):
        g.replay()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / replays / len(calls) * 1e3


def copies_for(nbytes: int, at_least: int = 4) -> int:
    """How many copies of an operand of this size make 1.5 GB, several times the memory-side cache."""
    return max(at_least, min(64, -(-(3 << 29) // max(1, nbytes))))


def decode_attention(args) -> None:
    nq, nkv, hd, P = args.heads, args.kv_heads, args.head_dim, args.page_size
    for B in args.batch:
        for ctx in args.context:
            pages_per = -(-ctx // P)
            kv_bytes = B * ctx * nkv * hd * 2 * 2
            nv = copies_for(kv_bytes, 8)
            n_pages = nv * B * pages_per
            k_pool = torch.randn(n_pages, nkv, P, hd, device=DEV).bfloat16()
            v_pool = torch.randn(n_pages, nkv, hd, P, device=DEV).bfloat16()
            tables = torch.randperm(n_pages).int().reshape(nv, B, pages_per).to(DEV)
            q = torch.randn(B, nq * hd, device=DEV).bfloat16()
            out = torch.empty_like(q)
            pos = torch.full((B,), ctx - 1, dtype=torch.int32, device=DEV)
            ent = torch.arange(B, dtype=torch.int32, device=DEV)
            groups = -(-(nq // nkv) // 16)
            auto = ops.decode_split(B, nkv, groups, ctx, hd)
            cells = []
            for splits, waves in [(0, 0)] + [(s, w) for w in (4, 8, 1) for s in (1, 2, 4, 8, 16, 32, 64)]:
                if splits * B * nkv * groups > 2048 or (hd == 256 and waves == 8):
                    continue
                calls = [(lambda v=v: ops.attention_decode_mfma(q, out, k_pool, v_pool, None, B, pos, ent, tables[v], P, nq,
                                                                nkv, hd, hd ** -0.5, 0, ctx, splits=splits, waves=waves))
                         for v in range(nv)]
                t = graph_time(calls)
                name = f"chosen {auto[1]}x{auto[0]}" if splits == 0 else f"{splits}x{waves}"
                cells.append(f"{name}: {t:.1f}")
            print(f"decode attention, batch {B}, context {ctx}, {nq}/{nkv} heads of {hd} ({kv_bytes / 1e6:.0f} MB of cache); "
                  f"us by splits x waves: " + "  ".join(cells), flush=True)
            del k_pool, v_pool


def prefill_attention(args) -> None:
    nq, nkv, hd, P = args.heads, args.kv_heads, args.head_dim, args.page_size
    for T in args.context:
        pages_per = -(-T // P)
        nv = 4
        n_pages = nv * pages_per
        k_pool = torch.randn(n_pages, nkv, P, hd, device=DEV).bfloat16()
        v_pool = torch.randn(n_pages, nkv, hd, P, device=DEV).bfloat16()
        tables = torch.randperm(n_pages).int().reshape(nv, 1, pages_per).to(DEV)
        q = torch.randn(T, nq * hd, device=DEV).bfloat16()
        out = torch.empty_like(q)
        pos = torch.arange(T, dtype=torch.int32, device=DEV)
        ent = torch.zeros(T, dtype=torch.int32, device=DEV)
        tile = ops.PREFILL_TILE
        tiles = torch.tensor([[i, min(tile, T - i)] for i in range(0, T, tile)], dtype=torch.int32, device=DEV)
        keys = [min(i + tile, T) for i in range(0, T, tile)]
        flops = 4 * nq * hd * T * (T + 1) / 2
        cells = []
        # 11, 12: the kernel that stages tiles in registers, where the one that loads them straight to LDS would run
        for halves in (0, 1, 2, 11, 12):
            calls = [(lambda v=v: ops.attention_prefill_mfma(q, out, k_pool, v_pool, tiles, tiles.shape[0], pos, ent, tables[v],
                                                             P, nq, nkv, hd, hd ** -0.5, 0, halves=halves,
                                                             keys_total=sum(keys), keys_max=max(keys)))
                     for v in range(nv)]
            t = graph_time(calls)
            name = {0: "chosen", 11: "staged, halves 1", 12: "staged, halves 2"}.get(halves, f"halves {halves}")
            cells.append(f"{name}: {t:.1f} us = {flops / t / 1e6:.0f} TFLOP/s")
        print(f"prompt attention, {T} tokens, {nq}/{nkv} heads of {hd}: " + "  ".join(cells), flush=True)
        del k_pool, v_pool


def projection(args) -> None:
    N, K = args.columns, args.inner
    w_bytes = N * K * 2
    nv = copies_for(w_bytes)
    ws = [torch.randn(N, K, device=DEV).bfloat16() * 0.02 for _ in range(nv)]
    gain = torch.ones(K, device=DEV)
    for M in args.rows:
        x = torch.randn(M, K, device=DEV).bfloat16()
        stream = torch.randn(M, K, device=DEV)
        resid = torch.zeros(M, N, device=DEV)
        cells = []

        def timed(name, make):
            try:
                make(0)()
            except ops.KernelError:
                return
            cells.append(f"{name}: {graph_time([make(v) for v in range(nv)]):.1f}")
        timed("library", lambda v: (lambda: torch.nn.functional.linear(x, ws[v])))
        if ops.gemm_skinny_supports(x, ws[0]):
            timed("skinny", lambda v: (lambda: ops.gemm_skinny(x, ws[v])))
            timed("skinny+add", lambda v: (lambda: ops.gemm_skinny_add(x, ws[v], resid)))
            if N % 2 == 0:
                timed("skinny+silu", lambda v: (lambda: ops.gemm_skinny_silu(x, ws[v])))
        if ops.gemm_skinny_normed_supports(stream, gain, ws[0]):
            timed("skinny+norm", lambda v: (lambda: ops.gemm_skinny_normed(stream, gain, 1e-6, ws[v])))
        if ops.gemm_rows_supports(x, ws[0]):
            timed("rows", lambda v: (lambda: ops.gemm_rows(x, ws[v])))
        if N % 2 == 0 and ops.gemm_rows_supports(x, ws[0], silu=True):
            timed("rows+silu", lambda v: (lambda: ops.gemm_rows(x, ws[v], silu=True)))
        if ops.gemm_partial_sums_supports(x, ws[0]):
            timed("partial sums", lambda v: (lambda: ops.gemm_partial_sums(x, ws[v])))
        if N % 2 == 0:
            timed("library+silu", lambda v: (lambda: ops.silu_mul(torch.nn.functional.linear(x, ws[v]))))
        floor = w_bytes / 8e12 * 1e6
        print(f"projection [{M}, {K}] x [{N}, {K}]^T ({w_bytes / 1e6:.0f} MB of weights, {floor:.1f} us at 8 TB/s); us: "
              + "  ".join(cells), flush=True)


TUNE_ROWS = [1, 4, 8, 9, 12, 16, 17, 24, 32, 33, 48, 64, 65, 96, 128, 192, 256]


def _ahead_up_to(rows, mine, others, start=0):
    """The row count r > ``start`` up to which taking ``mine`` instead of the best of ``others`` saves the most
    time in total over the measured row counts in (start, r] (``start`` if it never saves any).  A sum rather
    than "faster at every row count": one measurement that is off by its noise does not end a range."""
    best, best_gain, gain = start, 0.0, 0.0
    for r in rows:
        if r <= start:
            continue
        t = mine.get(r)
        rest = [o[r] for o in others if r in o]
        if t is None:
            break
        if not rest:
            continue
        gain += min(rest) - t
        if gain > best_gain + 1e-9:
            best, best_gain = r, gain
    return best


def derive_limits(times: dict, roles, columns: int, inner: int) -> dict:
    """The fields of :class:`dispatch.Limits` that the measured times of one matrix decide.  ``times`` is
    {kernel name: {rows: microseconds}} with rows as ints (see :func:`tune` for the names)."""
    rows = sorted({r for t in times.values() for r in t})
    get = lambda name: times.get(name, {})   # noqa: E731
    changes = {}
    if "store" in roles:
        changes["skinny"] = _ahead_up_to(rows, get("skinny"), [get("rows"), get("library")])
        changes["rows"] = _ahead_up_to(rows, get("rows"), [get("library"), get("partial sums>sum")], start=changes["skinny"])
        if changes["rows"] == changes["skinny"]:
            changes["rows"] = 0
        best = {r: min(t[r] for t in (get("skinny"), get("rows"), get("library")) if r in t) for r in rows}
        unfolded = {r: best[r] + get("norm")[r] for r in rows if r in get("norm")}
        changes["fold_norm"] = _ahead_up_to(rows, get("skinny+norm"), [unfolded])
        # above the rows the weight-streaming kernels take: partial sums and the kernel that adds them, against the library
        taken = max(changes["skinny"], changes["rows"])
        upto = _ahead_up_to(rows, get("partial sums>sum"), [get("library")], start=taken)
        changes["sums_from"], changes["sums_to"] = (taken + 1, upto) if upto > taken else (0, 0)
    if "silu" in roles:
        changes["silu_skinny"] = _ahead_up_to(rows, get("skinny+silu"), [get("rows+silu"), get("library+silu")])
        changes["silu_rows"] = _ahead_up_to(rows, get("rows+silu"), [get("library+silu")], start=changes["silu_skinny"])
        if changes["silu_rows"] == changes["silu_skinny"]:
            changes["silu_rows"] = 0
        best = {r: min(t[r] for t in (get("skinny+silu"), get("rows+silu"), get("library+silu")) if r in t) for r in rows}
        unfolded = {r: best[r] + get("norm")[r] for r in rows if r in get("norm")}
        changes["fold_norm"] = _ahead_up_to(rows, get("skinny+norm+silu"), [unfolded])
    if "stream" in roles:
        # up to 16 rows the few-rows kernel adds into the stream itself; the stacks serve the rows after that
        upto = _ahead_up_to(rows, get("partial sums>norm"), [get("library>norm")], start=16)
        changes["stacked_from"], changes["stacked_to"] = (17, upto) if upto > 16 else (0, 0)
    if "logits" in roles:
        changes["f32_skinny"] = _ahead_up_to(rows, get("skinny f32"), [get("library f32")])
    return changes


def tune(args) -> None:
    """Measure one matrix in its roles and write its limits.  Roles: ``store`` (a first projection, bfloat16
    out, with the norm before it), ``silu`` (gate|up: columns = 2 x intermediate), ``stream`` (a last
    projection, whose result goes into the residual stream), ``logits`` (32-bit out)."""
    N, K = args.columns, args.inner
    roles = set(args.roles)
    w_bytes = N * K * 2
    nv = copies_for(w_bytes)
    ws = [torch.randn(N, K, device=DEV).bfloat16() * 0.02 for _ in range(nv)]
    gain = torch.ones(K, device=DEV)
    times = {}

    def timed(name, rows, make):
        try:
            make(0)()
        except (ops.KernelError, RuntimeError):
            return
        times.setdefault(name, {})[rows] = round(graph_time([make(v) for v in range(nv)]), 2)
    for M in TUNE_ROWS:
        x = torch.randn(M, K, device=DEV).bfloat16()
        stream = torch.randn(M, K, device=DEV)
        skinny_ok = ops.gemm_skinny_supports(x, ws[0])
        if roles & {"store", "silu"}:
            # the norm kernel that a folded norm saves: the stream [M, K] to bfloat16 rows
            timed("norm", M, lambda v: (lambda: ops.add_rmsnorm(None, stream, gain, 1e-6, torch.bfloat16)))
        if "store" in roles:
            timed("library", M, lambda v: (lambda: torch.nn.functional.linear(x, ws[v])))
            if skinny_ok:
                timed("skinny", M, lambda v: (lambda: ops.gemm_skinny(x, ws[v])))
            if ops.gemm_skinny_normed_supports(stream, gain, ws[0]):
                timed("skinny+norm", M, lambda v: (lambda: ops.gemm_skinny_normed(stream, gain, 1e-6, ws[v])))
            if M <= ops.ROWS_MAX_ROWS and ops.gemm_rows_supports(x, ws[0]):
                timed("rows", M, lambda v: (lambda: ops.gemm_rows(x, ws[v])))
            if M > 16 and N % 4 == 0 and ops.gemm_partial_sums_supports(x, ws[0]):
                timed("partial sums>sum", M, lambda v: (lambda: ops.sum_stacks(ops.gemm_partial_sums(x, ws[v]))))
        if "silu" in roles:
            timed("library+silu", M, lambda v: (lambda: ops.silu_mul(torch.nn.functional.linear(x, ws[v]))))
            if skinny_ok:
                timed("skinny+silu", M, lambda v: (lambda: ops.gemm_skinny_silu(x, ws[v])))
            if ops.gemm_skinny_normed_supports(stream, gain, ws[0]):
                timed("skinny+norm+silu", M, lambda v: (lambda: ops.gemm_skinny_normed(stream, gain, 1e-6, ws[v], silu=True)))
            if M <= ops.ROWS_MAX_ROWS and ops.gemm_rows_supports(x, ws[0], silu=True):
                timed("rows+silu", M, lambda v: (lambda: ops.gemm_rows(x, ws[v], silu=True)))
        if "stream" in roles:
            resid = torch.zeros(M, N, device=DEV)
            gain_n = torch.ones(N, device=DEV)
            # the library's product, and the norm that adds it; against the stack and the norm that adds the stack
            timed("library>norm", M, lambda v: (lambda: ops.add_rmsnorm(torch.nn.functional.linear(x, ws[v]), resid, gain_n, 1e-6,
                                                                       torch.bfloat16)))
            if ops.gemm_partial_sums_supports(x, ws[0]):
                timed("partial sums>norm", M, lambda v: (lambda: ops.add_rmsnorm(ops.gemm_partial_sums(x, ws[v]), resid, gain_n, 1e-6,
                                                                                 torch.bfloat16)))
        if "logits" in roles:
            timed("library f32", M, lambda v: (lambda: torch.mm(x, ws[v].t(), out_dtype=torch.float32)))
            if skinny_ok and M <= 64:
                timed("skinny f32", M, lambda v: (lambda: ops.gemm_skinny(x, ws[v], out_dtype=torch.float32)))
        print(f"rows {M}: " + "  ".join(f"{k}: {v[M]}" for k, v in times.items() if M in v), flush=True)
    found = dispatch.default_limits(N, K)
    changes = derive_limits(times, roles, N, K)
    print(f"limits of {N}x{K}: {changes} (the size rules alone: "
          f"{ {k: getattr(found, k) for k in changes} })", flush=True)
    if not args.dry_run:
        dispatch.write_entry(N, K, changes)
        print(f"written to {dispatch.TABLE_PATH}", flush=True)


def sampling(args) -> None:
    """The sampling kernels on rows of normal logits (scale 3), per setting, both ways: rows cut into parts by a
    first kernel, and one block per row alone."""
    V = args.vocab
    settings = (("greedy", 0.0, -1, 1.0, 0.0), ("temperature 0.6", 0.6, -1, 1.0, 0.0),
                ("top-k 20, top-p 0.95", 0.6, 20, 0.95, 0.0), ("top-k 50", 0.8, 50, 1.0, 0.0),
                ("top-k 50, top-p 0.9, min-p 0.02", 0.8, 50, 0.9, 0.02), ("min-p 0.05", 0.8, -1, 1.0, 0.05),
                ("top-p 0.9 (these rows are flat: the long way)", 0.8, -1, 0.9, 0.0),
                ("top-p 0.9, rows of scale 12 (a nucleus of few values)", 0.8, -1, 0.9, 0.0))
    for B in args.rows:
        torch.manual_seed(0)
        flat_rows = torch.randn(B, V, device=DEV)
        lo, hi = torch.arange(B, dtype=torch.int32, device=DEV), torch.zeros(B, dtype=torch.int32, device=DEV)
        pos = torch.arange(B, dtype=torch.int32, device=DEV)
        out = torch.empty(B, dtype=torch.int32, device=DEV)
        for name, t, k, p, mp in settings:
            logits = flat_rows * (12 if "scale 12" in name else 3)
            T, K = torch.full((B,), t, device=DEV), torch.full((B,), k, dtype=torch.int32, device=DEV)
            P, MP = torch.full((B,), p, device=DEV), torch.full((B,), mp, device=DEV)
            cut = graph_time([lambda: ops.sample(logits, T, K, P, MP, lo, hi, pos, out, parts=True)])
            whole = graph_time([lambda: ops.sample(logits, T, K, P, MP, lo, hi, pos, out, parts=False)])
            print(f"sampling, {B} rows of {V} logits, {name}: rows cut into parts {cut:.1f} us, one block per row {whole:.1f} us",
                  flush=True)


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="ullm_amd.kernels.microbench", description=__doc__.split("\n\n")[0])
    sub = ap.add_subparsers(dest="what", required=True)
    ints = lambda s: [int(x) for x in s.split(",")]   # noqa: E731
    for name in ("decode-attention", "prefill-attention"):
        p = sub.add_parser(name)
        p.add_argument("--heads", type=int, default=32)
        p.add_argument("--kv-heads", type=int, default=8)
        p.add_argument("--head-dim", type=int, default=128)
        p.add_argument("--page-size", type=int, default=16)
        p.add_argument("--batch", type=ints, default=[1, 8, 64], help="comma-separated batch sizes (decode)")
        p.add_argument("--context", type=ints, default=[1100], help="comma-separated context lengths / prompt lengths")
    p = sub.add_parser("projection")
    p.add_argument("--columns", type=int, required=True, help="rows of the weight matrix (columns of the result)")
    p.add_argument("--inner", type=int, required=True)
    p.add_argument("--rows", type=ints, default=[1, 8, 16, 32, 64, 128], help="comma-separated numbers of rows of x")
    p = sub.add_parser("tune")
    p.add_argument("--columns", type=int, required=True, help="rows of the weight matrix (columns of the result)")
    p.add_argument("--inner", type=int, required=True)
    p.add_argument("--roles", type=lambda s: s.split(","), required=True,
                   help="comma-separated roles of the matrix: store, silu, stream, logits")
    p.add_argument("--dry-run", action="store_true", help="measure and print, leave the table as it is")
    p = sub.add_parser("sampling")
    p.add_argument("--vocab", type=int, default=151936)
    p.add_argument("--rows", type=ints, default=[1, 8, 64, 256], help="comma-separated numbers of rows of logits")
    args = ap.parse_args(argv)
    {"decode-attention": decode_attention, "prefill-attention": prefill_attention, "projection": projection,
     "tune": tune, "sampling": sampling}[args.what](args)
    return 0


if __name__ == "__main__":
    raise SystemExit(main())

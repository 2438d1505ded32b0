"""Which product kernel a projection takes, by its number of rows and its matrix.

Every choice between the hand-written product kernels and the library is a row limit: up to how many rows of
the batch a kernel is ahead for a matrix of ``columns`` x ``inner``.  The limits of a matrix come from a table
of measurements (``tuned_gfx950.json`` beside this file, written by
``python -m ullm_amd.kernels.microbench tune --columns N --inner K``), and for a matrix the table does not hold
from rules in terms of the matrix's size alone.  Parts ask :func:`limits`; none of them names a model or carries
a threshold of its own.  A limit only ever selects among kernels that compute the same function, and every
kernel's own ``*_supports`` check still decides whether it can take the operands at all, so a wrong or missing
entry costs time, never a result.
"""
from __future__ import annotations

import json
import os
from dataclasses import asdict, dataclass, fields
from typing import Dict, Optional

TABLE_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "tuned_gfx950.json")


@dataclass(frozen=True)
class Limits:
    """Row limits of one weight matrix [columns, inner] (for gate|up: columns = 2 x intermediate)."""
    # y = x W^T in bfloat16: the few-rows kernel up to ``skinny`` rows, then the rows kernel up to ``rows``
    # (0: never), then the library
    skinny: int = 16
    rows: int = 64
    # the RMS norm before the product folded into the few-rows kernel up to this many rows (asked where the product
    # before has not prepared the norm: a model's first layer, a part behind one that adds no result of its own)
    fold_norm: int = 8
    # silu(gate) * up on store: the few-rows kernel up to ``silu_skinny``, the rows kernel up to ``silu_rows``,
    # then the library product and the activation kernel
    silu_skinny: int = 16
    silu_rows: int = 64
    # a product whose result the next norm adds to the stream: as a stack of partial sums over slices of the
    # inner dimension from ``stacked_from`` to ``stacked_to`` rows (0, 0: never)
    stacked_from: int = 17
    stacked_to: int = 256
    # y = x W^T in bfloat16 above ``skinny`` and ``rows``: partial sums over slices of the inner dimension and a
    # kernel that adds them, from ``sums_from`` to ``sums_to`` rows (0, 0: never; only measured matrices have it)
    sums_from: int = 0
    sums_to: int = 0
    # 32-bit results (the logits head): the few-rows kernel up to here, then the library
    f32_skinny: int = 16


def default_limits(columns: int, inner: int) -> Limits:
    """The rules for a matrix that was not measured, in terms of its size alone.  They follow what the
    measured matrices (2 M to 780 M elements) have in common: the rows kernel needs enough columns to give
    every compute unit a block; a small matrix has few blocks to pay for 32-bit rows of X, so the norm stays
    folded in for every row count the kernel takes; gate|up keeps the few-rows kernel to 32 rows unless the
    matrix is very large, and the rows kernel to 128 rows from 12 288 result columns on; stacks of partial sums outweigh a matrix of a few M elements; the few-rows kernel
    with four tiles a block is ahead of the library up to 32 rows on matrices with very many columns."""
    weight = columns * inner
    return Limits(
        skinny=16,
        rows=64 if columns >= 2048 else 0,
        fold_norm=16 if weight <= (40 << 20) else 8,
        silu_skinny=32 if weight <= 200_000_000 else 16,
        silu_rows=(128 if columns // 2 >= 12288 else 64) if columns // 2 >= 2048 else 0,
        stacked_from=17 if weight >= (8 << 20) else 0,
        stacked_to=256 if weight >= (8 << 20) else 0,
        f32_skinny=32 if columns >= 65536 else 16)


_table: Optional[dict] = None


def _load() -> dict:
    global _table
    if _table is None:
        table: Dict[str, Limits] = {}
        if os.path.isfile(TABLE_PATH):
            with open(TABLE_PATH, "r", encoding="utf-8") as f:
                raw = json.load(f)
            names = {f.name for f in fields(Limits)}
            for key, entry in raw.get("matrices", {}).items():
                try:
                    columns, inner = (int(x) for x in key.split("x"))
                except ValueError:
                    raise ValueError(f"{TABLE_PATH}: key {key!r} is not COLUMNSxINNER") from None
                base = asdict(default_limits(columns, inner))
                base.update({k: int(v) for k, v in entry.items() if k in names})
                table[key] = Limits(**base)
        _table = table
    return _table


def limits(columns: int, inner: int) -> Limits:
    """The row limits of a weight matrix [columns, inner]: measured ones where the table has the matrix,
    the size rules otherwise."""
    table = _load()
    found = table.get((columns, inner))                    # by a tuple: this is asked for every projection of every step
    if found is None:
        found = table.get(f"{columns}x{inner}")
        if found is None:
            return default_limits(columns, inner)
        table[(columns, inner)] = found
    return found


def is_tuned(columns: int, inner: int) -> bool:
    return f"{columns}x{inner}" in _load()


def write_entry(columns: int, inner: int, fields_measured: Dict[str, int]) -> None:
    """Put the measured limits of one matrix into the table file (used by ``microbench tune``); fields that
    were not measured for it are left to the size rules."""
    global _table
    names = {f.name for f in fields(Limits)}
    unknown = set(fields_measured) - names
    if unknown:
        raise KeyError(f"no such limits: {sorted(unknown)}")
    raw = {"device": "gfx950", "matrices": {}}
    if os.path.isfile(TABLE_PATH):
        with open(TABLE_PATH, "r", encoding="utf-8") as f:
            raw = json.load(f)
    entry = raw.setdefault("matrices", {}).setdefault(f"{columns}x{inner}", {})
    entry.update({k: int(v) for k, v in fields_measured.items()})
    with open(TABLE_PATH, "w", encoding="utf-8") as f:
        json.dump(raw, f, indent=1, sort_keys=True)
        f.write("\n")
    _table = None

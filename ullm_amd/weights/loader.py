"""Binds safetensors tensors to a model's declared weights by name.

The reference streams every tensor of every ``*.safetensors`` file to ``load_weights`` and silently
skips names it does not know; parameters that never receive a tensor stay uninitialised
(ullm/model_loader.py:25-49, ullm/models/qwen3.py:300-336).  Here the file's names and shapes are
compared with what the parts declare *before* anything is copied, and one error lists every
missing tensor, every unexpected tensor and every wrong shape.

Dtypes: matrices are held in the compute dtype (bfloat16, or float32 in the 32-bit mode, where a
bfloat16 checkpoint widens exactly); tensors a part marks ``keep_fp32`` (norm gains, biases) are
held in float32 whatever they were stored as; integer tensors become int32.
"""
from __future__ import annotations

import glob
import os
from dataclasses import dataclass
from typing import Dict, List, Tuple

import torch
from safetensors import safe_open

from ..parts import PartEnv, WeightDecl

# names some exporters add that carry no weights of the model
IGNORABLE_SUFFIXES = ("rotary_emb.inv_freq",)


class WeightError(RuntimeError):
    """The checkpoint does not match the model; the message lists every problem."""


def checkpoint_index(model_dir: str) -> Dict[str, Tuple[str, Tuple[int, ...], str]]:
    """{tensor name: (file, shape, dtype string)} over every *.safetensors in the folder."""
    files = sorted(glob.glob(os.path.join(model_dir, "*.safetensors")))
    if not files:
        raise WeightError(f"{model_dir}: no *.safetensors file in the model folder")
    index: Dict[str, Tuple[str, Tuple[int, ...], str]] = {}
    for path in files:
        with safe_open(path, framework="pt") as f:
            for name in f.keys():
                sl = f.get_slice(name)
                if name in index:
                    raise WeightError(f"tensor {name!r} appears in both {index[name][0]} and {path}")
                index[name] = (path, tuple(sl.get_shape()), str(sl.get_dtype()))
    return index


def _final_dtype(decl: WeightDecl, stored: torch.dtype, compute: torch.dtype) -> torch.dtype:
    if not stored.is_floating_point:
        return torch.int32
    if decl.keep_fp32:
        return torch.float32
    return compute


@dataclass
class MergedTensor:
    """A matrix that several declared tensors are the rows of (q | k | v, gate | up)."""
    name: str
    shape: Tuple[int, ...]
    pieces: List[WeightDecl]          # by rising row_offset; together they cover every row once


def unique_decls(decls: List[WeightDecl]) -> Dict[str, WeightDecl]:
    declared: Dict[str, WeightDecl] = {}
    for d in decls:
        if d.name in declared and declared[d.name].shape != d.shape:
            raise WeightError(f"two parts declare {d.name!r} with shapes {declared[d.name].shape} and {d.shape}")
        declared.setdefault(d.name, d)
    return declared


def merged_tensors(decls: List[WeightDecl]) -> Dict[str, MergedTensor]:
    """{merged name: MergedTensor} of every matrix the declarations put together from pieces."""
    by_name: Dict[str, List[WeightDecl]] = {}
    for d in unique_decls(decls).values():
        if d.merged_into is not None:
            by_name.setdefault(d.merged_into, []).append(d)
    out = {}
    for name, pieces in by_name.items():
        pieces.sort(key=lambda d: d.row_offset)
        rows = 0
        for d in pieces:
            if d.row_offset != rows or tuple(d.shape[1:]) != tuple(pieces[0].shape[1:]) or d.keep_fp32 != pieces[0].keep_fp32:
                raise WeightError(f"the pieces of {name!r} do not tile its rows: {[(x.name, x.row_offset, x.shape) for x in pieces]}")
            rows += d.shape[0]
        out[name] = MergedTensor(name, (rows,) + tuple(pieces[0].shape[1:]), pieces)
    return out


def check_against(decls: List[WeightDecl], index) -> None:
    """One error that lists every missing tensor, every unexpected tensor and every wrong shape.
    A merged matrix may come as its pieces (the usual export) or whole under its merged name (the
    reference takes both, ullm/layers/linear.py:359-379,473-485), not as a mixture."""
    declared = unique_decls(decls)
    merged = merged_tensors(decls)
    missing, wrong = [], []
    for name, d in declared.items():
        if name in index:
            if tuple(index[name][1]) != tuple(d.shape):
                wrong.append(f"  {name}  checkpoint has {list(index[name][1])}, model needs {list(d.shape)}")
            continue
        if d.alias_of is not None and d.alias_of in index:
            continue
        if d.merged_into is not None and d.merged_into in index:
            continue
        missing.append(f"  {name}  expected shape {list(d.shape)}")
    unexpected = []
    for n in sorted(index):
        if n in declared or n.endswith(IGNORABLE_SUFFIXES):
            continue
        if n in merged:
            m = merged[n]
            if tuple(index[n][1]) != tuple(m.shape):
                wrong.append(f"  {n}  checkpoint has {list(index[n][1])}, model needs {list(m.shape)}")
            both = [d.name for d in m.pieces if d.name in index]
            if both:
                unexpected.append(f"  {n}  shape {list(index[n][1])}  (the checkpoint also holds its pieces {both})")
            continue
        unexpected.append(f"  {n}  shape {list(index[n][1])}")
    if missing or wrong or unexpected:
        parts = ["checkpoint does not match the model:"]
        if missing:
            parts.append(f"missing tensors ({len(missing)}):\n" + "\n".join(missing))
        if unexpected:
            parts.append(f"unexpected tensors ({len(unexpected)}):\n" + "\n".join(unexpected))
        if wrong:
            parts.append(f"wrong shapes ({len(wrong)}):\n" + "\n".join(wrong))
        raise WeightError("\n".join(parts))


def bind_tensors(part, tensors: Dict[str, torch.Tensor], env: PartEnv) -> None:
    """Bind one part (and the parts below it) from tensors that are already in memory, named as in a
    checkpoint: pieces of merged matrices are put together here as ``load_weights`` does from files."""
    from ..parts import walk
    decls = [d for p in walk(part) for d in p.weights()]
    out = {n: t.to(env.device) for n, t in tensors.items()}
    for m in merged_tensors(decls).values():
        if m.name not in out:
            out[m.name] = torch.cat([out.pop(d.name) for d in m.pieces], dim=0)
    for p in walk(part):
        p.bind(out, env)


def load_weights(model, model_dir: str, env: PartEnv) -> None:
    """Check the folder against ``model.weight_decls()``, bring every tensor to ``env.device`` in its
    final dtype and hand them to the parts.  A merged matrix is allocated once and its pieces are
    copied from the file straight into its rows, so nothing is held twice on the device."""
    decls = model.weight_decls()
    index = checkpoint_index(model_dir)
    check_against(decls, index)
    declared = unique_decls(decls)
    merged = merged_tensors(decls)
    # what to read from each file: (name in the file, declaration it fills or None for a whole merged matrix)
    by_file: Dict[str, List[Tuple[str, object]]] = {}
    aliases: List[WeightDecl] = []
    for d in declared.values():
        if d.name in index:
            by_file.setdefault(index[d.name][0], []).append((d.name, d))
        elif d.merged_into is None:
            aliases.append(d)
    for m in merged.values():
        if m.name in index:
            by_file.setdefault(index[m.name][0], []).append((m.name, m))
    tensors: Dict[str, torch.Tensor] = {}
    for path, items in by_file.items():
        with safe_open(path, framework="pt") as f:
            for name, what in items:
                t = f.get_tensor(name)
                if isinstance(what, MergedTensor):
                    tensors[name] = t.to(device=env.device, dtype=_final_dtype(what.pieces[0], t.dtype, env.dtype))
                elif what.merged_into is None:
                    tensors[name] = t.to(device=env.device, dtype=_final_dtype(what, t.dtype, env.dtype))
                else:
                    m = merged[what.merged_into]
                    buf = tensors.get(m.name)
                    if buf is None:
                        buf = tensors[m.name] = torch.empty(m.shape, dtype=_final_dtype(what, t.dtype, env.dtype),
                                                            device=env.device)
                    buf[what.row_offset:what.row_offset + what.shape[0]].copy_(t)     # widens or narrows on the way
    for d in aliases:
        tensors[d.name] = tensors[d.alias_of]          # tied: the same storage, no copy
    model.bind(tensors, env)

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


def check_against(decls: List[WeightDecl], index) -> None:
    declared = {}
    for d in decls:
        if d.name in declared and declared[d.name].shape != d.shape:
            raise WeightError(f"two parts declare {d.name!r} with shapes {declared[d.name].shape} and {d.shape}")
        declared.setdefault(d.name, d)
    missing, wrong = [], []
    for name, d in declared.items():
        if name not in index:
            if d.alias_of is not None and d.alias_of in index:
                continue
            missing.append(f"  {name}  expected shape {list(d.shape)}")
        elif tuple(index[name][1]) != tuple(d.shape):
            wrong.append(f"  {name}  checkpoint has {list(index[name][1])}, model needs {list(d.shape)}")
    unexpected = [f"  {n}  shape {list(index[n][1])}" for n in sorted(index)
                  if n not in declared and not n.endswith(IGNORABLE_SUFFIXES)]
    if missing or wrong or unexpected:
        parts = ["checkpoint does not match the model:"]
        if missing:
            parts.append(f"missing tensors ({len(missing)}):\n" + "\n".join(missing))
        if unexpected:
            parts.append(f"unexpected tensors ({len(unexpected)}):\n" + "\n".join(unexpected))
        if wrong:
            parts.append(f"wrong shapes ({len(wrong)}):\n" + "\n".join(wrong))
        raise WeightError("\n".join(parts))


def load_weights(model, model_dir: str, env: PartEnv) -> None:
    """Check the folder against ``model.weight_decls()``, copy every tensor to ``env.device`` in its
    final dtype and hand them to the parts."""
    decls = model.weight_decls()
    index = checkpoint_index(model_dir)
    check_against(decls, index)
    by_file: Dict[str, List[WeightDecl]] = {}
    aliases: List[WeightDecl] = []
    seen = set()
    for d in decls:
        if d.name in seen:
            continue
        seen.add(d.name)
        if d.name in index:
            by_file.setdefault(index[d.name][0], []).append(d)
        else:
            aliases.append(d)
    tensors: Dict[str, torch.Tensor] = {}
    for path, ds in by_file.items():
        with safe_open(path, framework="pt") as f:
            for d in ds:
                t = f.get_tensor(d.name)
                tensors[d.name] = t.to(device=env.device, dtype=_final_dtype(d, t.dtype, env.dtype))
    for d in aliases:
        tensors[d.name] = tensors[d.alias_of]          # tied: the same storage, no copy
    model.bind(tensors, env)

"""Random weights from a configuration and a seed (the reference has no such mode).

``write_random_model`` writes a model folder (config.json, model.safetensors) that any loader of
the format can read: tensors are drawn on the CPU in the order the parts declare them from one
seeded generator, matrices and embeddings N(0, std), norm gains 1 + N(0, std), in float32, then
stored in the requested dtype.  ``bind_random_weights`` draws straight on the device instead, for
sizes where a file would only cost time (benchmarks).
"""
from __future__ import annotations

import json
import os
from typing import Dict, Mapping, Optional

import torch
from safetensors.torch import save_file

from ..models import build_model
from ..parts import PartEnv

_STORE = {"bfloat16": torch.bfloat16, "float32": torch.float32}


def _draw(decl, std: float, gen: torch.Generator, device) -> torch.Tensor:
    t = torch.empty(decl.shape, dtype=torch.float32, device=device).normal_(0.0, std, generator=gen)
    if decl.init == "gain":
        t += 1.0
    return t


def write_random_model(config: Mapping, out_dir: str, seed: int, std: Optional[float] = None,
                       dtype: str = "bfloat16") -> str:
    """Write ``out_dir/config.json`` and ``out_dir/model.safetensors``; returns ``out_dir``."""
    if dtype not in _STORE:
        raise ValueError(f"storage dtype {dtype!r}: choose bfloat16 or float32")
    config = dict(config)
    config.setdefault("torch_dtype", dtype)
    _, model = build_model(config)
    sigma = model.plan.init_std if std is None else float(std)
    gen = torch.Generator(device="cpu").manual_seed(int(seed))
    tensors: Dict[str, torch.Tensor] = {}
    for d in model.weight_decls():
        if d.name in tensors or d.alias_of is not None:
            continue                                    # a tied head is not stored
        tensors[d.name] = _draw(d, sigma, gen, "cpu").to(_STORE[dtype]).contiguous()
    os.makedirs(out_dir, exist_ok=True)
    with open(os.path.join(out_dir, "config.json"), "w", encoding="utf-8") as f:
        json.dump(config, f, indent=1)
    save_file(tensors, os.path.join(out_dir, "model.safetensors"), metadata={"format": "pt"})
    return out_dir


def bind_random_weights(model, env: PartEnv, seed: int, std: Optional[float] = None,
                        store_dtype: str = "bfloat16") -> None:
    """Draw every declared tensor on ``env.device`` (own seeded generator) and bind the model.
    Matrices are drawn in ``store_dtype`` and then brought to the compute dtype, as a checkpoint
    stored in that dtype would be: the same seed gives the bfloat16 and the float32 engine the same
    weights (the float32 one holds them widened exactly).  Tensors a part keeps in 32-bit are drawn
    in 32-bit.  Pieces of a merged matrix are drawn straight into its rows."""
    from .loader import merged_tensors, unique_decls
    if store_dtype not in _STORE:
        raise ValueError(f"storage dtype {store_dtype!r}: choose bfloat16 or float32")
    sigma = model.plan.init_std if std is None else float(std)
    gen = torch.Generator(device=env.device).manual_seed(int(seed))
    decls = model.weight_decls()
    merged = merged_tensors(decls)
    tensors: Dict[str, torch.Tensor] = {}
    pending_alias = []
    for d in unique_decls(decls).values():
        if d.alias_of is not None:
            pending_alias.append(d)
            continue
        final = torch.float32 if d.keep_fp32 else env.dtype
        drawn = torch.float32 if d.keep_fp32 else _STORE[store_dtype]
        if d.merged_into is not None:
            m = merged[d.merged_into]
            buf = tensors.get(m.name)
            if buf is None:
                buf = tensors[m.name] = torch.empty(m.shape, dtype=final, device=env.device)
            target = buf[d.row_offset:d.row_offset + d.shape[0]]
        else:
            target = tensors[d.name] = torch.empty(d.shape, dtype=final, device=env.device)
        if drawn == final:
            target.normal_(0.0, sigma, generator=gen)          # in place: no second copy of a large matrix
        else:
            target.copy_(torch.empty(d.shape, dtype=drawn, device=env.device).normal_(0.0, sigma, generator=gen))
        if d.init == "gain":
            target += 1.0
    for d in pending_alias:
        tensors[d.name] = tensors[d.alias_of]
    model.bind(tensors, env)


def main(argv=None) -> int:
    """``python -m ullm_amd.weights.random_init --config config.json --out DIR --seed 0``"""
    import argparse
    ap = argparse.ArgumentParser(prog="ullm_amd.weights.random_init",
                                 description="Write a model folder with seeded random weights for a config.json")
    ap.add_argument("--config", required=True, help="config.json of the architecture (its own keys)")
    ap.add_argument("--out", required=True, help="folder to write config.json and model.safetensors into")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--std", type=float, default=None, help="standard deviation (default: the config's initializer_range)")
    ap.add_argument("--dtype", default="bfloat16", choices=sorted(_STORE))
    args = ap.parse_args(argv)
    with open(args.config, encoding="utf-8") as f:
        config = json.load(f)
    print(write_random_model(config, args.out, args.seed, args.std, args.dtype))
    return 0


if __name__ == "__main__":
    raise SystemExit(main())

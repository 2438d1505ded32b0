"""From a model folder to a model with weights on the device (reference:
ullm/core/model_runner.py:185-231: registry lookup, build in the model dtype, stream the weights)."""
from __future__ import annotations

import logging

import torch

from ..config.engine_config import normalize_dtype
from ..config.model_config import ConfigError, read_config_json
from ..kernels import build as kernel_build
from ..models import build_model
from ..parts import PartEnv
from ..weights.loader import load_weights

logger = logging.getLogger("ullm_amd")
TORCH_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32}


def make_env(dtype: str, device: str, context_len: int) -> PartEnv:
    dev = torch.device(device)
    if dev.type != "cuda":
        raise RuntimeError(f"device {device!r}: this engine runs its HIP kernels on a GPU only")
    if not torch.cuda.is_available():
        raise RuntimeError("no GPU is visible to torch; the engine has no other code path")
    # the 32-bit mode must not be served by reduced-precision matrix modes anywhere
    torch.backends.cuda.matmul.allow_tf32 = False
    torch.backends.cudnn.allow_tf32 = False
    return PartEnv(dev, TORCH_DTYPES[normalize_dtype(dtype)], int(context_len))


def context_within_model(cfg, context_len: int, strict: bool = True) -> int:
    """``context_len`` checked against the positions the model is defined for (a typed configuration's
    ``max_position_embeddings``, where it has one).  The reference builds its rotary table with that many rows
    (ullm/models/qwen3.py:142) and fails on a position past them.  An engine with a longer context is refused
    when it is built.  Not ``strict`` (trace replay, whose number is the size of a pool and whose traces are
    given): the angles of later positions follow from the same formula, and that is said once."""
    limit = getattr(cfg, "max_position_embeddings", None)
    if limit is None or context_len <= limit:
        return int(context_len)
    if strict:
        raise ConfigError(f"context_len={context_len} exceeds the model's max_position_embeddings={limit}: positions "
                          f"past it have no defined encoding (use --context-len {limit} or less)")
    logger.warning("positions up to %d are allowed for, past the model's max_position_embeddings=%d: their rotation "
                   "angles continue the same formula, the reference's table ends there", context_len, limit)
    return int(context_len)


def load_model(model_dir: str, dtype: str, device: str, context_len: int, strict_context: bool = True):
    """(typed config, model with bound weights, env)."""
    config_dict = read_config_json(model_dir)
    cfg, model = build_model(config_dict)
    env = make_env(dtype, device, context_within_model(cfg, context_len, strict_context))
    load_weights(model, model_dir, env)
    return cfg, model, env


def random_model(spec: str, dtype: str, device: str, context_len: int):
    """(typed config, model with random weights drawn on the device, env) for a specification
    ``NAME[:SEED]`` / ``CONFIG.JSON[:SEED]`` (see :func:`ullm_amd.config.parse_random_weights`)."""
    from ..config.engine_config import parse_random_weights
    from ..weights.random_init import bind_random_weights
    config_dict, seed = parse_random_weights(spec)
    cfg, model = build_model(config_dict)
    env = make_env(dtype, device, context_within_model(cfg, context_len))
    bind_random_weights(model, env, seed)
    return cfg, model, env

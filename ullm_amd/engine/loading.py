"""From a model folder to a model with weights on the device (reference:
ullm/core/model_runner.py:185-231: registry lookup, build in the model dtype, stream the weights)."""
from __future__ import annotations

import torch

from ..config.engine_config import normalize_dtype
from ..config.model_config import read_config_json
from ..kernels import build as kernel_build
from ..models import build_model
from ..parts import PartEnv
from ..weights.loader import load_weights

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


def load_model(model_dir: str, dtype: str, device: str, context_len: int):
    """(typed config, model with bound weights, env)."""
    config_dict = read_config_json(model_dir)
    cfg, model = build_model(config_dict)
    env = make_env(dtype, device, context_len)
    load_weights(model, model_dir, env)
    return cfg, model, env


def random_model(spec: str, dtype: str, device: str, context_len: int):
    """(typed config, model with random weights drawn on the device, env) for a specification
    ``NAME[:SEED]`` / ``CONFIG.JSON[:SEED]`` (see :func:`ullm_amd.config.parse_random_weights`)."""
    from ..config.engine_config import parse_random_weights
    from ..weights.random_init import bind_random_weights
    config_dict, seed = parse_random_weights(spec)
    cfg, model = build_model(config_dict)
    env = make_env(dtype, device, context_len)
    bind_random_weights(model, env, seed)
    return cfg, model, env

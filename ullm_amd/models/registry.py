"""One registry from an architecture's name (config.json "architectures") to its typed
configuration and its plan.  Reference: ullm/models/registry.py:3-5 and the lookup with its error
in ullm/core/model_runner.py:186-194.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Dict, Mapping

from ..config.model_config import ConfigError
from .model import Model, ModelPlan


@dataclass(frozen=True)
class Architecture:
    name: str
    config_from_dict: Callable[[Mapping], object]   # config.json dict -> typed config
    plan: Callable[[object], ModelPlan]             # typed config -> model plan


MODEL_REGISTRY: Dict[str, Architecture] = {}


def register_architecture(name: str, config_from_dict, plan) -> None:
    MODEL_REGISTRY[name] = Architecture(name, config_from_dict, plan)


def resolve_architecture(config_dict: Mapping) -> Architecture:
    archs = config_dict.get("architectures") or []
    for a in archs:
        if a in MODEL_REGISTRY:
            return MODEL_REGISTRY[a]
    raise ConfigError(f"Model arch {list(archs)} not supported. Registered: {sorted(MODEL_REGISTRY)}")


def build_model(config_dict: Mapping):
    """(typed config, Model) for a config.json dict; no weights bound yet."""
    arch = resolve_architecture(config_dict)
    cfg = arch.config_from_dict(config_dict)
    return cfg, Model(arch.plan(cfg))

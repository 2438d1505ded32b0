"""Typed model configuration read from the architecture's own config.json keys.

The reference hands config.json to a library class and reads attributes where it needs
them (ullm/config.py:43, ullm/models/qwen3.py:139-157,207,224,268,
ullm/core/model_runner.py:31-73).  Here the keys are parsed once into a frozen
dataclass; every size and constant the model uses comes from this object.
"""
from __future__ import annotations

import json
import os
from dataclasses import asdict, dataclass, fields
from typing import Any, Mapping


class ConfigError(ValueError):
    """A config.json that cannot be turned into a model configuration."""


_REQUIRED = object()


def _take(d: Mapping[str, Any], key: str, kind, default=_REQUIRED):
    if key not in d or d[key] is None:
        if default is _REQUIRED:
            raise ConfigError(f"config.json: required key '{key}' is missing")
        return default
    v = d[key]
    try:
        if kind is bool:
            if not isinstance(v, (bool, int)):
                raise TypeError
            return bool(v)
        if kind is int:
            if isinstance(v, bool) or int(v) != v:
                raise TypeError
            return int(v)
        if kind is float:
            return float(v)
        if kind is str:
            if not isinstance(v, str):
                raise TypeError
            return v
    except (TypeError, ValueError):
        pass
    raise ConfigError(f"config.json: key '{key}' has value {v!r}, expected {kind.__name__}")


@dataclass(frozen=True)
class Qwen3Config:
    """Keys of a Qwen3 dense config.json.

    Defaults follow the reference: ``head_dim = hidden_size // num_attention_heads``
    (ullm/models/qwen3.py:78, ullm/core/model_runner.py:60-63), ``rope_theta = 1e6``
    (qwen3.py:144), ``attention_bias = False`` (qwen3.py:146); ``rms_norm_eps`` is read
    without a default (qwen3.py:145).  ``tie_word_embeddings`` and the sliding-window
    keys are not read by the reference (it always owns a separate lm_head,
    qwen3.py:267-270, and never masks by distance); they are read here so that a tied
    checkpoint binds and a windowed config chooses a windowed mixer layer by layer.
    """

    architectures: tuple
    vocab_size: int
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    max_position_embeddings: int
    rms_norm_eps: float
    rope_theta: float
    attention_bias: bool
    tie_word_embeddings: bool
    hidden_act: str
    use_sliding_window: bool
    sliding_window: int
    max_window_layers: int
    layer_types: tuple            # per layer "full_attention" / "sliding_attention", or () where config.json has no list
    torch_dtype: str
    eos_token_id: int             # the first stop id config.json names (-1: none)
    eos_token_ids: tuple          # all of them: config.json may hold a list
    initializer_range: float

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "Qwen3Config":
        archs = d.get("architectures")
        if not isinstance(archs, (list, tuple)) or not archs:
            raise ConfigError("config.json: required key 'architectures' is missing or empty")
        hidden = _take(d, "hidden_size", int)
        nq = _take(d, "num_attention_heads", int)
        nkv = _take(d, "num_key_value_heads", int, nq)
        if nq <= 0 or nkv <= 0 or nq % nkv != 0:
            raise ConfigError(
                f"config.json: num_attention_heads={nq} must be a positive multiple of "
                f"num_key_value_heads={nkv}")
        head_dim = _take(d, "head_dim", int, None)
        if head_dim is None:
            if hidden % nq != 0:
                raise ConfigError(
                    f"config.json: no 'head_dim' and hidden_size={hidden} is not a multiple "
                    f"of num_attention_heads={nq}")
            head_dim = hidden // nq
        use_window = _take(d, "use_sliding_window", bool, False)
        window = _take(d, "sliding_window", int, 0)
        layers = _take(d, "num_hidden_layers", int)
        max_window_layers = _take(d, "max_window_layers", int, layers)
        if use_window and window <= 0:
            raise ConfigError("config.json: use_sliding_window is true but 'sliding_window' "
                              "is missing or not positive")
        kinds = d.get("layer_types")
        if kinds is None:
            kinds = ()
        elif (not isinstance(kinds, (list, tuple)) or len(kinds) != layers
              or any(k not in ("full_attention", "sliding_attention") for k in kinds)):
            raise ConfigError(f"config.json: layer_types={kinds!r} must name 'full_attention' or 'sliding_attention' "
                              f"for each of the {layers} layers")
        elif "sliding_attention" in kinds and not use_window:
            raise ConfigError("config.json: layer_types names sliding_attention layers but use_sliding_window is "
                              "not true: which keys such a layer sees is not defined")
        act = _take(d, "hidden_act", str, "silu")
        if act != "silu":
            raise ConfigError(f"config.json: hidden_act={act!r}; this architecture's "
                              "feed-forward is SwiGLU (silu)")
        dtype = d.get("dtype") or d.get("torch_dtype") or "bfloat16"
        if not isinstance(dtype, str):
            raise ConfigError(f"config.json: dtype={dtype!r} is not a string")
        eos = d.get("eos_token_id")
        eos_ids = tuple(eos) if isinstance(eos, (list, tuple)) else (() if eos is None else (eos,))
        for e in eos_ids:
            if isinstance(e, bool) or not isinstance(e, int) or e < 0:
                raise ConfigError(f"config.json: eos_token_id={eos!r} must be a token id or a list of token ids")
        # The reference builds its rotation angles from rope_theta alone (ullm/models/qwen3.py:97-102,
        # ullm/layers/rotary_embedding.py:52-75) and so does this engine: a config that asks for scaled
        # angles would run with wrong ones, so it is refused rather than served quietly.
        scaling = d.get("rope_scaling")
        if scaling is not None:
            kind = scaling.get("rope_type", scaling.get("type")) if isinstance(scaling, Mapping) else scaling
            if kind not in (None, "default"):
                raise ConfigError(f"config.json: rope_scaling={scaling!r} is not supported (only absent, null or "
                                  "type 'default': the rotation angles come from rope_theta alone)")
        cfg = cls(
            architectures=tuple(str(a) for a in archs),
            vocab_size=_take(d, "vocab_size", int),
            hidden_size=hidden,
            num_hidden_layers=layers,
            num_attention_heads=nq,
            num_key_value_heads=nkv,
            head_dim=head_dim,
            intermediate_size=_take(d, "intermediate_size", int),
            max_position_embeddings=_take(d, "max_position_embeddings", int),
            rms_norm_eps=_take(d, "rms_norm_eps", float),
            rope_theta=_take(d, "rope_theta", float, 1000000.0),
            attention_bias=_take(d, "attention_bias", bool, False),
            tie_word_embeddings=_take(d, "tie_word_embeddings", bool, False),
            hidden_act=act,
            use_sliding_window=use_window,
            sliding_window=window,
            max_window_layers=max_window_layers,
            layer_types=tuple(kinds),
            torch_dtype=dtype,
            eos_token_id=int(eos_ids[0]) if eos_ids else -1,
            eos_token_ids=tuple(int(e) for e in eos_ids),
            initializer_range=_take(d, "initializer_range", float, 0.02),
        )
        for name in ("vocab_size", "hidden_size", "num_hidden_layers", "head_dim",
                     "intermediate_size", "max_position_embeddings"):
            if getattr(cfg, name) <= 0:
                raise ConfigError(f"config.json: '{name}' must be positive, got {getattr(cfg, name)}")
        if cfg.head_dim % 2 != 0:
            raise ConfigError(f"config.json: head_dim={cfg.head_dim} must be even for rotary pairs")
        if cfg.rms_norm_eps < 0:
            raise ConfigError("config.json: 'rms_norm_eps' must not be negative")
        return cfg

    def to_dict(self) -> dict:
        d = asdict(self)
        d["architectures"] = list(self.architectures)
        d["eos_token_ids"] = list(self.eos_token_ids)
        if self.layer_types:
            d["layer_types"] = list(self.layer_types)
        else:
            del d["layer_types"]
        return d

    def window_of_layer(self, layer: int) -> int:
        """Keys a query of this layer may look back over, itself included; 0 = all.  A per-layer list in
        config.json decides where there is one, else the layers from ``max_window_layers`` on have the window."""
        if not self.use_sliding_window:
            return 0
        if self.layer_types:
            return self.sliding_window if self.layer_types[layer] == "sliding_attention" else 0
        return self.sliding_window if layer >= self.max_window_layers else 0


def read_config_json(model_dir: str) -> dict:
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"{model_dir}: no config.json in the model folder")
    with open(path, "r", encoding="utf-8") as f:
        try:
            d = json.load(f)
        except json.JSONDecodeError as e:
            raise ConfigError(f"{path}: not valid JSON ({e})") from None
    if not isinstance(d, dict):
        raise ConfigError(f"{path}: top level must be an object")
    return d


def config_field_names(cls) -> list:
    return [f.name for f in fields(cls)]

"""Engine configuration in the reference's manner.

Field names and meanings follow ullm/config.py:9-25 where the reference has them
(``model``, ``gpu_memory_utilization``, ``max_bs``, ``context_len``, ``enforce_eager``,
``log_level``, and ``tp_size``/``pp_size`` which must stay 1 on this single-GPU engine).
What the reference lacks (pages larger than a token, a token budget, prompt portions,
a 32-bit mode, a seed) is added beside them.
"""
from __future__ import annotations

import argparse
import json
import os
from dataclasses import dataclass, field
from typing import List, Optional

from .model_config import ConfigError

_DTYPES = {
    "bfloat16": "bfloat16", "bf16": "bfloat16",
    "float32": "float32", "fp32": "float32", "float": "float32",
}


def normalize_dtype(name: str) -> str:
    key = str(name).lower().replace("torch.", "")
    if key not in _DTYPES:
        raise ConfigError(f"dtype {name!r} is not supported: choose bfloat16 or float32")
    return _DTYPES[key]


PRESET_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "presets")


def preset_names() -> List[str]:
    """Named sizes ``random_weights`` knows: config.json files that ship with the package."""
    return sorted(f[:-5] for f in os.listdir(PRESET_DIR) if f.endswith(".json"))


def parse_random_weights(spec: str):
    """(config.json dict, seed) of a ``NAME[:SEED]`` / ``PATH[:SEED]`` specification."""
    name, seed = spec, 0
    if ":" in spec and spec.rsplit(":", 1)[1].lstrip("-").isdigit():
        name, seed = spec.rsplit(":", 1)[0], int(spec.rsplit(":", 1)[1])
    path = os.path.join(PRESET_DIR, name.lower() + ".json") if name.lower() in preset_names() else name
    if not os.path.isfile(path):
        raise ConfigError(f"random weights {spec!r}: {name!r} is neither a config.json nor one of {preset_names()}")
    with open(path, "r", encoding="utf-8") as f:
        try:
            config = json.load(f)
        except json.JSONDecodeError as e:
            raise ConfigError(f"{path}: not valid JSON ({e})") from None
    return config, seed


@dataclass
class EngineConfig:
    model: Optional[str] = None                 # folder with config.json and *.safetensors
    gpu_memory_utilization: float = 0.9         # share of free device memory the cache may take
    max_bs: int = 50                            # most live requests (= request slots)
    tp_size: int = 1
    pp_size: int = 1
    context_len: int = 2048                     # most tokens (prompt + generated) of a request
    enforce_eager: bool = False                 # True: never replay decode steps from HIP graphs
    disable_async_scheduling: bool = False      # True: schedule a step only after the one before has ended
    log_level: str = "info"
    nccl_port: int = 29500                      # the reference's option; one GPU opens no port
    device_ids: Optional[List[int]] = None      # the reference's option; exactly one id here (sets ``device``)
    profile: bool = False                       # True: LLM.profile("start" | "stop") records a torch profiler trace
    profile_dir: str = "./profiles"             # where those traces are written
    # -- beyond the reference ------------------------------------------------------
    dtype: str = "bfloat16"                     # "bfloat16" | "float32" (whole model in true 32-bit)
    page_size: int = 16                         # tokens per cache page.  16 is what the decode attention kernel reads in one
                                                # piece: values lie transposed in a page, [head_dim, page_size], and a
                                                # wave takes 16 keys of 16 dims per load, so with longer pages it uses a
                                                # part of every line it fetches (measured 1.2x slower at 32, 2x at 64)
    num_pages: Optional[int] = None             # pages of every cache group; None: from memory
    max_num_batched_tokens: int = 2048          # token budget of one step
    max_prefill_chunk: int = 2048               # longest prompt portion given to one request per step
    enable_prefix_cache: bool = False           # share whole pages of equal prompt prefixes
    seed: int = 0                               # default seed for requests that bring none
    device: str = "cuda:0"
    # instead of ``model``: NAME[:SEED] or PATH[:SEED], a named size (see ``preset_names``) or a config.json,
    # whose weights are drawn on the device from the seed (default 0)
    random_weights: Optional[str] = None

    def __post_init__(self):
        self.dtype = normalize_dtype(self.dtype)
        if (self.model is None) == (self.random_weights is None):
            raise ConfigError("give either a model folder (model) or a random-weights specification, not both or neither")
        if self.tp_size != 1 or self.pp_size != 1:
            raise ConfigError("this engine runs on one GPU: tp_size and pp_size must be 1")
        if self.device_ids is not None:
            if len(self.device_ids) != 1:
                raise ConfigError(f"this engine runs on one GPU: device_ids={self.device_ids} must name exactly one")
            self.device = f"cuda:{int(self.device_ids[0])}"
        if self.max_bs < 1:
            raise ConfigError("max_bs must be at least 1")
        if self.context_len < 1:
            raise ConfigError("context_len must be at least 1")
        if self.page_size < 1 or (self.page_size & (self.page_size - 1)) != 0:
            raise ConfigError(f"page_size={self.page_size} must be a power of two")
        if self.max_num_batched_tokens < 1 or self.max_prefill_chunk < 1:
            raise ConfigError("max_num_batched_tokens and max_prefill_chunk must be at least 1")
        if not (0.0 < self.gpu_memory_utilization <= 1.0):
            raise ConfigError("gpu_memory_utilization must lie in (0, 1]")

    @staticmethod
    def add_cli_args(parser: argparse.ArgumentParser) -> None:
        """Options with the reference's names and defaults (ullm/entrypoints/api_server.py:130-183)
        followed by this engine's own."""
        parser.add_argument("--model", type=str, default=None, help="Model folder")
        parser.add_argument("--random-weights", type=str, default=None, metavar="SPEC",
                            help="instead of --model: NAME[:SEED] or CONFIG.JSON[:SEED], random weights drawn on the "
                                 f"device; names: {', '.join(preset_names())}")
        parser.add_argument("--gpu-memory-utilization", type=float, default=0.9,
                            help="GPU memory utilization")
        parser.add_argument("--max-bs", type=int, default=50, help="Maximum batch size")
        parser.add_argument("--tp-size", type=int, default=1, help="Tensor parallel size (must be 1)")
        parser.add_argument("--pp-size", type=int, default=1, help="Pipeline parallel size (must be 1)")
        parser.add_argument("--context-len", type=int, default=2048,
                            help="Max context length of the model")
        parser.add_argument("--enforce-eager", action="store_true",
                            help="Enforce eager execution, disable HIP graphs")
        parser.add_argument("--nccl-port", type=int, default=29500, help="Unused with one GPU (kept for the reference's callers)")
        parser.add_argument("--device-ids", type=lambda v: [int(x) for x in v.split(",")], default=None,
                            help="The GPU to use (one id)")
        parser.add_argument("--profile", action="store_true", help="Enable torch profiler traces (LLM.profile)")
        parser.add_argument("--profile-dir", type=str, default="./profiles", help="Directory for profiler traces")
        parser.add_argument("--disable-async-scheduling", action="store_true",
                            help="Do not schedule the next step while the device runs the current one")
        parser.add_argument("--log-level", type=str, default="info", help="Log level for the engine")
        parser.add_argument("--dtype", type=str, default="bfloat16", help="bfloat16 or float32")
        parser.add_argument("--page-size", type=int, default=16, help="Tokens per cache page")
        parser.add_argument("--num-pages", type=int, default=None,
                            help="Cache pages per group (default: from free memory)")
        parser.add_argument("--max-num-batched-tokens", type=int, default=2048,
                            help="Token budget of one step")
        parser.add_argument("--max-prefill-chunk", type=int, default=2048,
                            help="Longest prompt portion per request and step")
        parser.add_argument("--enable-prefix-cache", action="store_true",
                            help="Share cache pages between equal prompt prefixes")
        parser.add_argument("--seed", type=int, default=0, help="Default sampling seed")

    @staticmethod
    def from_args(args: argparse.Namespace) -> "EngineConfig":
        return EngineConfig(
            model=args.model,
            gpu_memory_utilization=args.gpu_memory_utilization,
            max_bs=args.max_bs,
            tp_size=args.tp_size,
            pp_size=args.pp_size,
            context_len=args.context_len,
            enforce_eager=args.enforce_eager,
            disable_async_scheduling=args.disable_async_scheduling,
            nccl_port=args.nccl_port, device_ids=args.device_ids, profile=args.profile, profile_dir=args.profile_dir,
            log_level=args.log_level,
            dtype=args.dtype,
            page_size=args.page_size,
            num_pages=args.num_pages,
            max_num_batched_tokens=args.max_num_batched_tokens,
            max_prefill_chunk=args.max_prefill_chunk,
            enable_prefix_cache=args.enable_prefix_cache,
            seed=args.seed,
            random_weights=getattr(args, "random_weights", None),
        )

    def generation_defaults(self) -> dict:
        """Sampling defaults from generation_config.json beside the model, for the keys the
        reference copies (ullm/config.py:46-67): temperature, top_k, top_p, min_p."""
        out = {}
        path = os.path.join(self.model, "generation_config.json") if self.model else ""
        if path and os.path.isfile(path):
            with open(path, "r", encoding="utf-8") as f:
                d = json.load(f)
            for key in ("temperature", "top_k", "top_p", "min_p"):
                if d.get(key) is not None:
                    out[key] = d[key]
        return out

from .model import Choice, Model, ModelPlan
from .registry import MODEL_REGISTRY, Architecture, build_model, register_architecture, resolve_architecture
from . import qwen3  # noqa: F401  (registers Qwen3ForCausalLM)

__all__ = ["Choice", "Model", "ModelPlan", "MODEL_REGISTRY", "Architecture", "build_model",
           "register_architecture", "resolve_architecture"]

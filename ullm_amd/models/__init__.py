from .model import Choice, Model, ModelPlan
from .registry import MODEL_REGISTRY, Architecture, build_model, register_architecture, resolve_architecture
from . import qwen3  # noqa: F401  (registers Qwen3ForCausalLM)
from . import pamopel  # noqa: F401  (registers Pamopel)
from . import ziferax  # noqa: F401  (registers Ziferax)
from . import dovisun  # noqa: F401  (registers Dovisun)
from . import kumudra  # noqa: F401  (registers Kumudra)

__all__ = ["Choice", "Model", "ModelPlan", "MODEL_REGISTRY", "Architecture", "build_model",
           "register_architecture", "resolve_architecture"]

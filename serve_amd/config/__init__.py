from .engine import EngineConfig  # noqa: F401
from .llama import ConfigError, Llama3RopeScaling, LlamaConfig  # noqa: F401
from .spec import LayerSpec, ModelSpec, PartSpec, RunEntry  # noqa: F401

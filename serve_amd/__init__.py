"""serve_amd: a single-GPU inference engine for the dense Llama decoder on AMD MI355X (gfx950).

    from serve_amd import load_model, generate, Request
"""
from .config.engine import EngineConfig  # noqa: F401
from .config.llama import LlamaConfig, Llama3RopeScaling  # noqa: F401
from .registry import (get_architecture, known_architectures, load_config,  # noqa: F401
                       register_architecture, register_part)

__all__ = ["EngineConfig", "LlamaConfig", "Llama3RopeScaling", "Engine", "Request", "load_model",
           "generate", "get_architecture", "known_architectures", "load_config",
           "register_architecture", "register_part"]


def __getattr__(name):
    # the engine pulls in the kernels; keep `import serve_amd` light for configuration-only use
    if name in ("Engine", "Request", "load_model", "generate"):
        from .engine import engine as _engine
        return getattr(_engine, name)
    raise AttributeError(name)

from .registry import ModelSpec, get_spec, known_models, read_model_dir, register, resolve
from .runtime import RuntimeConfig, parse_dtype

__all__ = ["ModelSpec", "RuntimeConfig", "get_spec", "known_models", "parse_dtype", "read_model_dir", "register",
           "resolve"]

"""kestrel_amd: a single-GPU inference engine for AMD MI355X (gfx950).

``from kestrel_amd import InferenceEngine, RuntimeConfig``; ``python -m kestrel_amd --help``.
"""

from .config import RuntimeConfig, get_spec, known_models

__version__ = "0.1.0"


def __getattr__(name):
    if name in ("InferenceEngine", "EngineResult", "EngineMetrics", "StepEntry", "ModelRunner"):
        from . import engine
        return getattr(engine, name)
    raise AttributeError(name)


__all__ = ["InferenceEngine", "RuntimeConfig", "get_spec", "known_models"]

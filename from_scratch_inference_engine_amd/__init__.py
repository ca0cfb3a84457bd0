"""Importable name of the engine.

The sources live in the folder ``from-scratch-inference-engine-_amd/`` beside this one; a
hyphen cannot appear in an ``import`` statement, so this package points its search path there.
``import from_scratch_inference_engine_amd.cache`` loads
``from-scratch-inference-engine-_amd/cache/__init__.py`` and so on.
"""

from pathlib import Path as _Path

__version__ = "0.1.0"

_SOURCES = _Path(__file__).resolve().parent.parent / "from-scratch-inference-engine-_amd"
if not _SOURCES.is_dir():  # pragma: no cover - broken checkout
    raise ImportError(f"engine sources not found at {_SOURCES}")
__path__ = [str(_SOURCES)]

_PUBLIC = {
    "LLM": ("engine.llm", "LLM"),
    "GenerationConfig": ("engine.llm", "GenerationConfig"),
    "Engine": ("engine.engine", "Engine"),
    "SeqStatus": ("engine.scheduler", "SeqStatus"),
    "SamplingParams": ("sampling.params", "SamplingParams"),
    "load_model": ("models.registry", "load_model"),
    "load_config": ("models.registry", "load_config"),
    "write_random_model": ("weights.random_init", "write_random_model"),
}


def __getattr__(name):
    """Lazy public names, so that ``import ...cache`` alone does not import torch code paths
    it does not need."""
    if name in _PUBLIC:
        import importlib

        module, attr = _PUBLIC[name]
        value = getattr(importlib.import_module(f"{__name__}.{module}"), attr)
        globals()[name] = value
        return value
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")

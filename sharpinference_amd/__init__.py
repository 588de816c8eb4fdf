"""sharpinference_amd: a small, whole inference engine for one GPU (MI355X, gfx950).

``Engine`` opens a model folder (config.json + model.safetensors) or builds random weights
from a configuration and a seed, steps mixed batches through hand-written HIP kernels from a
paged cache, and generates under continuous batching.
"""
from .config.base import ConfigError, ModelConfig, load_config  # noqa: F401
from .registry import build_model, register_architecture, registered_architectures  # noqa: F401
from .sampling.params import SamplingParams  # noqa: F401


def __getattr__(name):
    if name in ("Engine", "GenerateChunk", "GenerationResult", "StepEntry"):
        from . import engine as _e

        return getattr(_e, name)
    raise AttributeError(name)

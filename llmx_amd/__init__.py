"""llmx_amd: a small, whole inference engine for one MI355X.

Everything between a request's tokens and its next token: typed configuration and an architecture registry, weights
from safetensors by name or from a seed, layers assembled from parts, a paged cache with block tables, one step
function over mixed batches, a scheduler, sampling, and hand-written gfx950 kernels underneath.
Importing the package touches neither the GPU nor the kernel library; both are needed from the first `Engine` on.
"""

from .config import ConfigError, MiniMaxM3Config
from .weights import RandomInit, WeightsError

__version__ = "0.1.0"


def __getattr__(name):
    # the engine side imports torch's GPU pieces and the kernel library: load it on first use
    if name in ("Engine", "StepEntry", "StepError"):
        from . import engine
        return getattr(engine, name)
    if name in ("generate", "Generator"):
        from .engine import generation
        return getattr(generation, name)
    if name in ("Scheduler", "Request"):
        from .engine import scheduler
        return getattr(scheduler, name)
    if name == "SamplingParams":
        from .sampling import SamplingParams
        return SamplingParams
    if name == "write_random_model":
        from .weights.folder import write_random_model
        return write_random_model
    raise AttributeError(f"module 'llmx_amd' has no attribute {name!r}")


__all__ = ["ConfigError", "MiniMaxM3Config", "RandomInit", "WeightsError", "Engine", "StepEntry", "StepError", "generate",
           "Generator", "SamplingParams", "Scheduler", "Request", "write_random_model"]

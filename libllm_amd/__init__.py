"""libllm_amd: a small Llama-family inference library for one AMD MI355X GPU."""
from .errors import (CacheError, ConfigError, KernelError, LlmError, RequestError,  # noqa: F401
                     WeightError)

__version__ = "0.1.0"


def __getattr__(name):
    # the entry-point classes import torch and the engine; load them on first use
    if name in ("Model", "Device", "ControlToken", "Chunk", "Completion", "StepEntry", "SamplingParams"):
        from . import api
        from .engine import StepEntry
        from .sampling import SamplingParams
        return {"StepEntry": StepEntry, "SamplingParams": SamplingParams}.get(name) or getattr(api, name)
    raise AttributeError(name)

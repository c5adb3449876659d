"""Error types of the library.  Every failure a caller can cause raises one of these."""


class LlmError(Exception):
    """Base class."""


class ConfigError(LlmError):
    """A config.json key is missing, has the wrong type, or an unsupported value."""


class WeightError(LlmError):
    """The tensors of a model file do not match what the model declares."""


class CacheError(LlmError):
    """No free slot or page, a request held twice, released twice, or grown past its limit."""


class KernelError(LlmError):
    """The HIP extension is missing, cannot be built, or was given operands it refuses."""


class RequestError(LlmError):
    """A step or generation request that the engine cannot run (bad token id, empty prompt)."""


class ReplayMismatch(LlmError):
    """Work recorded into a graph did not, replayed, give the bits it gives when queued directly."""

from .sampler import TOP_K_MAX, Sampler, SamplingParams  # noqa: F401

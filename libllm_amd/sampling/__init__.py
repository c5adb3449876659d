from .sampler import TOP_K_MAX, PendingTokens, Sampler, SamplingParams  # noqa: F401

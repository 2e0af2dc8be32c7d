from .sampler import RequestSampling, Sampler, SamplingParams, initial_state, xorshift64   # noqa: F401

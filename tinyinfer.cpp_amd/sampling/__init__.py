from .sampler import SamplingParams, Sampler, uniform, DEFAULT_TOP_K

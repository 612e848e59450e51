from .sampler import SamplingParams, Sampler, uniform_for

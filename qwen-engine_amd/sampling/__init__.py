from .sampler import Sampler, SamplingParams, uniform_for

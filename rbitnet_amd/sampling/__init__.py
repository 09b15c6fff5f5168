from .sampler import Sampler, uniform

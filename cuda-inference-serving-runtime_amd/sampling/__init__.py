from .sampler import Sampler, uniform01

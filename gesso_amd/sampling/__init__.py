from .sampler import Sampler, choose

from .sampler import Sampler, request_seed

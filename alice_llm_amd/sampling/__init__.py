from .sampler import Sampler, splitmix64, uniform, GREEDY_BELOW

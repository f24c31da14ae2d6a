from .sampler import GREEDY_EPS, Sampler, mix_key

__all__ = ["GREEDY_EPS", "Sampler", "mix_key"]

from .sampler import GenerationConfig, GREEDY, Sampler, XorShift64Star, MAX_TOP_K

__all__ = ["GenerationConfig", "GREEDY", "Sampler", "XorShift64Star", "MAX_TOP_K"]

from .config import GREEDY, SamplingConfig, defaults
from .sampler import XorShift64Star, make_rng, pack_settings, sample_rows

__all__ = ["GREEDY", "SamplingConfig", "defaults", "XorShift64Star", "make_rng",
           "pack_settings", "sample_rows"]

from .config import GREEDY, MAX_DEVICE_TOP_K, SamplingConfig, defaults
from .sampler import XorShift64Star, draw_from_candidates, host_candidates, make_rng, sample_rows

__all__ = ["GREEDY", "MAX_DEVICE_TOP_K", "SamplingConfig", "defaults", "XorShift64Star", "draw_from_candidates",
           "host_candidates", "make_rng", "sample_rows"]

from .config import GREEDY, SamplingConfig, defaults
from .sampler import XorShift64Star, draw_from_candidates, host_candidates, make_rng, pack_settings, sample_rows

__all__ = ["GREEDY", "SamplingConfig", "defaults", "XorShift64Star", "draw_from_candidates", "host_candidates", "make_rng",
           "pack_settings", "sample_rows"]

from .rng import XorShift64Star, stream_seed
from .sampler import Sampler, SamplingOptions, SequenceSampling

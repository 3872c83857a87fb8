from .params import SAMPLING_EPS, SamplingParams, TokenLogprob
from .rng import rand_f32, fresh_seed
from .sampler import Sampler

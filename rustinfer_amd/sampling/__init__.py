from .params import SamplingParams
from .sampler import Sampler, fresh_seed, splitmix64, uniform_draw

from .params import STRATEGIES, SamplingConfig
from .sampler import Sampler, uniform_at

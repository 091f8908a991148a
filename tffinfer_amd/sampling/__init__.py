from .params import STRATEGIES, SamplingConfig
from .sampler import Sampler, SeenTokens, uniform_at

from .params import SamplingConfig, read_generation_config
from .sampler import Sampler, PendingTokens, uniform

from .params import REPEAT_LAST_N, SamplingParams
from .rng import mix64, stream, stream_i64, uniform
from .sampler import Sampler

__all__ = ["REPEAT_LAST_N", "SamplingParams", "Sampler", "mix64", "stream", "stream_i64", "uniform"]

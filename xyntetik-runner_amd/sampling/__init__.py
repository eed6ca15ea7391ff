from .params import SamplingParams, SamplerState, xorshift64, RECENT_WINDOW
from .sampler import Sampler

__all__ = ["SamplingParams", "SamplerState", "xorshift64", "RECENT_WINDOW", "Sampler"]

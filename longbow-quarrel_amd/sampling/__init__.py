"""Greedy, temperature, top-k, top-p and repetition-penalty sampling on the device."""
from .params import SamplingParams
from .sampler import NonFiniteLogits, Sampler
from .state import RECENT, SamplerState, sequence_key

__all__ = ["SamplingParams", "NonFiniteLogits", "Sampler", "RECENT", "SamplerState", "sequence_key"]

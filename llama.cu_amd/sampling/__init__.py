"""Greedy, temperature, top-k and top-p sampling."""
from .params import GREEDY, TOP_K_ALL, SamplingParams
from .sampler import Sampler, argmax, sample_rows, token_logprobs, uniform

__all__ = ["GREEDY", "TOP_K_ALL", "SamplingParams", "Sampler", "argmax", "sample_rows", "token_logprobs", "uniform"]

from .params import GREEDY_EPS, SamplingParams, TokenLogprobs

__all__ = ["GREEDY_EPS", "SamplingParams", "TokenLogprobs"]

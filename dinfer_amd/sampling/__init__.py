from .params import GREEDY_EPS, SamplingParams

__all__ = ["GREEDY_EPS", "SamplingParams"]

"""dinfer_amd: a small, whole LLM inference engine for one MI355X GPU."""
from .config import EngineOptions
from .sampling.params import SamplingParams, TokenLogprobs

__version__ = "0.1.0"
__all__ = ["Engine", "EngineOptions", "SamplingParams", "TokenLogprobs"]


def __getattr__(name):
    if name == "Engine":
        from .engine.engine import Engine
        return Engine
    raise AttributeError(name)

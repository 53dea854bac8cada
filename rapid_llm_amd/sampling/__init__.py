from .logprobs import PositionLogprobs
from .params import SamplingParams
from .rng import uniform_draw

__all__ = ["SamplingParams", "PositionLogprobs", "Sampler", "RowSampling", "uniform_draw"]


def __getattr__(name):
    if name in ("Sampler", "RowSampling"):
        from . import sampler

        return getattr(sampler, name)
    raise AttributeError(name)

from .params import SamplingParams

__all__ = ["SamplingParams", "Sampler", "NonFiniteLogits"]


def __getattr__(name):
    if name in ("Sampler", "NonFiniteLogits"):
        from . import sampler
        return getattr(sampler, name)
    raise AttributeError(name)

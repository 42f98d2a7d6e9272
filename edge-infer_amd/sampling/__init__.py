from .params import MAX_TOP_K, SamplingParams

__all__ = ["MAX_TOP_K", "SamplingParams", "Sampler"]


def __getattr__(name):
    if name == "Sampler":
        from .sampler import Sampler
        return Sampler
    raise AttributeError(name)

from .params import SamplingParams, fresh_seed, uniform_for

__all__ = ["SamplingParams", "Sampler", "fresh_seed", "uniform_for"]


def __getattr__(name):
    if name == "Sampler":          # needs the GPU library; imported on demand
        from .sampler import Sampler
        return Sampler
    raise AttributeError(name)

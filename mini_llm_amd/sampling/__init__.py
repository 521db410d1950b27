from .params import SamplingParams

__all__ = ["SamplingParams", "Sampler"]


def __getattr__(name):
    if name == "Sampler":  # needs torch and the kernels; the parameters alone do not
        from .sampler import Sampler

        return Sampler
    raise AttributeError(name)

from .config import SamplingConfig

__all__ = ["SamplingConfig", "Sampler"]


def __getattr__(name):
    if name == "Sampler":                    # needs the kernels; the options do not
        from .sampler import Sampler
        return Sampler
    raise AttributeError(name)

from .params import CLI_DEFAULTS, SamplingParams, stream_state

__all__ = ["CLI_DEFAULTS", "SamplingParams", "stream_state", "Sampler"]


def __getattr__(name):
    if name == "Sampler":
        from .sampler import Sampler
        return Sampler
    raise AttributeError(name)

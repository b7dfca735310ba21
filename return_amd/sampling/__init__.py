from .params import SamplingParams, UniformStream, ends_with_stop

__all__ = ["SamplingParams", "UniformStream", "ends_with_stop"]

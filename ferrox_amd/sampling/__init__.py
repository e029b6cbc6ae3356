from .sampler import SamplingParams, XorShift64, sample_rows

__all__ = ["SamplingParams", "XorShift64", "sample_rows"]

from .sampler import SamplingParams, XorShift64, launch_sample_rows, sample_rows

__all__ = ["SamplingParams", "XorShift64", "launch_sample_rows", "sample_rows"]

from tokenmill_amd.sampling.sampler import Sampler, SamplingParams, uniform_from_counter

__all__ = ["Sampler", "SamplingParams", "uniform_from_counter"]

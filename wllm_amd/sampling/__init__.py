from wllm_amd.sampling.params import SamplingParams
from wllm_amd.sampling.sampler import Sampler

__all__ = ["SamplingParams", "Sampler"]

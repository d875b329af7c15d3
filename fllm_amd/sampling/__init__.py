from .params import SamplingParams
from .sampler import SampleRequest, Sampler, pack_rows

__all__ = ["SamplingParams", "SampleRequest", "Sampler", "pack_rows"]

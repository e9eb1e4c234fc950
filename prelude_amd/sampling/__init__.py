from .sampler import DEFAULT_SEED, RequestSampler, SamplingParams, sample_rows

__all__ = ["DEFAULT_SEED", "RequestSampler", "SamplingParams", "sample_rows"]

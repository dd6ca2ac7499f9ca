from .pending import PendingToken, PendingTokens
from .sampler import Rng, Sampler, SamplerConfig, greedy_pending, host_sample, sample_rows, sample_rows_pending

__all__ = ["PendingToken", "PendingTokens", "Rng", "Sampler", "SamplerConfig", "greedy_pending", "host_sample", "sample_rows",
           "sample_rows_pending"]

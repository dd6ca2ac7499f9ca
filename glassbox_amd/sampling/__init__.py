from .sampler import Rng, Sampler, SamplerConfig, host_sample, sample_rows

__all__ = ["Rng", "Sampler", "SamplerConfig", "host_sample", "sample_rows"]

from .sampler import Rng, Sampling, sample_host

__all__ = ["Rng", "Sampling", "sample_host"]

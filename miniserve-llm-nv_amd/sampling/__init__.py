from .sampler import NonFiniteLogitsError, Sampler, StagedSample

__all__ = ["NonFiniteLogitsError", "Sampler", "StagedSample"]

from .rng import Rng
from .sampler import MAX_LOGIT_BIAS, RECENT_WINDOW, BatchSampler, RowRequest, SamplingParams, seeded_state

__all__ = ["Rng", "MAX_LOGIT_BIAS", "RECENT_WINDOW", "BatchSampler", "RowRequest", "SamplingParams", "seeded_state"]

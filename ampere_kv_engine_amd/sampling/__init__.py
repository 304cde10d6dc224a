from .sampler import NO_TOKEN, Sampler, SamplingParams, SlotSampler

__all__ = ["NO_TOKEN", "Sampler", "SamplingParams", "SlotSampler"]

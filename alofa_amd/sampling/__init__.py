from .sampler import LOGIT_FLOOR, SampleParams, Sampler, SplitMix64, pick_from, softmax_f64

__all__ = ["LOGIT_FLOOR", "SampleParams", "Sampler", "SplitMix64", "pick_from", "softmax_f64"]

from .sampler import SampleParams, XorShift64Star, apply_bias_and_penalties, argmax, logit_change_entries, sample

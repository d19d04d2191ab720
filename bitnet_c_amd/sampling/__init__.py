from .sampler import SamplingParams, SequenceSampler, XorShift64Star, sample_batch

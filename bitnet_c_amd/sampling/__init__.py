from .sampler import PendingTokens, SamplingParams, SequenceSampler, XorShift64Star, sample_batch, start_sampling

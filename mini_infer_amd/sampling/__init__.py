from mini_infer_amd.sampling.params import SamplingParams
from mini_infer_amd.sampling.sampler import sample_batch, sample_from_slots, sample_tokens

__all__ = ["SamplingParams", "sample_batch", "sample_from_slots", "sample_tokens"]

from .sampler import Rng, Sampler, SamplingParams, argmax_row, pick_rows, random_seed

__all__ = ["Rng", "Sampler", "SamplingParams", "argmax_row", "pick_rows", "random_seed"]

from .sampler import PendingRowPicks, Rng, Sampler, SamplingParams, argmax_row, pick_rows, random_seed

__all__ = ["PendingRowPicks", "Rng", "Sampler", "SamplingParams", "argmax_row", "pick_rows", "random_seed"]

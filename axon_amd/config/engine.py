"""The engine's own settings: what the model's config.json does not decide."""
from __future__ import annotations

from dataclasses import dataclass

from .base import ConfigError

DTYPES = {"bfloat16": "bfloat16", "bf16": "bfloat16", "float32": "float32", "fp32": "float32", "f32": "float32"}


def dtype_name(name: str) -> str:
    try:
        return DTYPES[name]
    except KeyError:
        raise ConfigError(f"dtype {name!r} is not one of bfloat16, float32") from None


@dataclass
class EngineConfig:
    """`dtype`: "bfloat16" (what serving uses) or "float32" (every product and sum in true
    32-bit).  `page_size`: positions in one cache page.  `num_pages`: pages in each cache
    group's pool; 0 sizes the pool from `max_cache_tokens`, and that being 0 too, from the
    free device memory times `memory_fraction`.  `max_seqs`: live requests at most (rows of
    the block tables and state slots).  `max_batch_tokens`: tokens one step may carry.
    `max_seq_len`: positions a request may reach (0: the model's max_position_embeddings).
    `use_graphs`: replay pure decode steps from captured HIP graphs."""
    dtype: str = "bfloat16"
    page_size: int = 64
    num_pages: int = 0
    max_cache_tokens: int = 0
    memory_fraction: float = 0.85
    max_seqs: int = 64
    max_batch_tokens: int = 2048
    max_seq_len: int = 0
    use_graphs: bool = True
    shuffle_pages_seed: int = -1

    def __post_init__(self):
        self.dtype = dtype_name(self.dtype)
        if self.page_size < 1:
            raise ConfigError(f"page_size {self.page_size} must be at least 1")
        if self.max_seqs < 1 or self.max_batch_tokens < 1:
            raise ConfigError("max_seqs and max_batch_tokens must be at least 1")

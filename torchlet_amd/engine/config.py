"""The engine's own sizes, as one typed object.

What the model folder does not say and the engine has to be told: how the cache is cut into pages and
how many there are, how many requests live at a time, how many tokens a step may hold, how long a
sequence may get.  The reference derives these in its engine's constructor from three arguments
(/root/reference/src/torchlet/v10_triton_paged_gqa/engine.py:39-59: pages per request from
``max_position_embeddings``, pool = slots * pages per request + 1 unless given, cache dtype = the
model's); here they are fields with the same meanings, and the Python entry point, the command line,
the trace replay and the benchmark all build their step function from one of these.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, replace


@dataclass(frozen=True)
class EngineConfig:
    page_size: int = 16                  # tokens per cache page (the reference's kv_block_size)
    num_pages: int | None = None         # pages of the pool, the sentinel included (max_num_blocks); None: see resolve()
    memory_fraction: float = 0.8         # with num_pages None: the share of free GPU memory the pool may take at most
    max_slots: int = 4                   # most requests live at a time (max_decode_slots)
    max_tokens_per_step: int = 2048      # token budget of a step: decode tokens first, prompt portions with the rest
    max_model_len: int | None = None     # most positions of a sequence; None: the model's max_position_embeddings
    dtype: str | None = None             # compute dtype: bfloat16, or float32 for the true 32-bit path; None: the model folder's
    kv_dtype: str | None = None          # element type of the cache pages; None: the compute dtype (no other is built)
    use_graphs: bool = False             # decode-only steps replay a captured HIP graph
    lookahead: bool = True               # the engine enqueues a decode step before it has read the tokens of the one before
    seed: int = 0                        # sampler seed
    bounded_steps: bool = True           # steps never exceed max_tokens_per_step: pools of windowed groups are sized by it

    def __post_init__(self):
        for name in ("page_size", "max_slots", "max_tokens_per_step"):
            v = getattr(self, name)
            if not isinstance(v, int) or isinstance(v, bool) or v <= 0:
                raise ValueError(f"{name} must be a positive integer, got {v!r}")
        if self.num_pages is not None and self.num_pages < 2:
            raise ValueError("num_pages counts the sentinel page: it must be at least 2")
        if self.max_model_len is not None and self.max_model_len <= 0:
            raise ValueError("max_model_len must be positive")
        if not 0.0 < self.memory_fraction <= 1.0:
            raise ValueError("memory_fraction must lie in (0, 1]")
        if self.dtype is not None and _canonical(self.dtype) not in ("bfloat16", "float32"):
            raise ValueError(f"compute dtype must be bfloat16 or float32, got {self.dtype!r}")
        if self.kv_dtype is not None and self.dtype is not None and _canonical(self.kv_dtype) != _canonical(self.dtype):
            raise ValueError(f"cache pages of {self.kv_dtype} under a {self.dtype} engine are not built: the cache has the compute dtype")

    def model_len(self, model_max_positions: int) -> int:
        """Most positions of a sequence: the model's own limit, or less if asked."""
        return model_max_positions if self.max_model_len is None else min(self.max_model_len, model_max_positions)

    def resolve(self, model_max_positions: int, bytes_per_page: int, free_bytes: int | None) -> "EngineConfig":
        """The same configuration with ``num_pages`` filled in: every slot can hold a sequence of the greatest
        length (``max_slots * ceil(model_len / page_size) + 1``, the reference's rule), but no more than
        ``memory_fraction`` of the free memory."""
        if self.num_pages is not None:
            return self
        pages = self.max_slots * math.ceil(self.model_len(model_max_positions) / self.page_size) + 1
        if free_bytes is not None and bytes_per_page > 0:
            pages = min(pages, int(free_bytes * self.memory_fraction) // bytes_per_page)
        return replace(self, num_pages=max(2, pages))


def _canonical(name: str) -> str:
    return {"bf16": "bfloat16", "fp32": "float32", "f32": "float32"}.get(str(name).lower(), str(name).lower())

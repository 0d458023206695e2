"""Engine knobs (pages, admission, prompt portions), validated on construction.

Names, defaults and meanings follow flow_engine/config.py:68-92 where the
reference has them. Left out: `attention` (one backend here) and `draft_*`
(speculation is not built). Added: `dtype`, `max_step_tokens` (token budget of
one step), `adaptive_chunk` (the reference's wall-clock feedback on the prompt
portion, off by default so runs are reproducible), `use_graphs` and `lookahead`.
"""
from __future__ import annotations

from dataclasses import dataclass


@dataclass(frozen=True)
class EngineConfig:
    block_size: int = 16            # tokens per page
    kv_blocks: int = 256            # physical pages per cache group
    max_context: int = 2048         # prompt + generated tokens per request
    max_active: int = 4             # admitted requests
    max_queue: int = 32             # waiting requests
    prefill_chunk: int = 256        # largest prompt portion in one step
    min_prefill_chunk: int = 16     # smallest portion the feedback may choose
    target_step_ms: float = 50.0    # feedback target for one step
    prefix_cache: bool = True       # reuse full pages of equal prompt prefixes
    dtype: str = "bfloat16"         # "bfloat16" | "float32"
    max_step_tokens: int = 0        # 0: max_active + prefill_chunk
    adaptive_chunk: bool = False    # flow_engine/engine.py:262-268 feedback controller
    use_graphs: bool = True         # replay decode-only steps from HIP graphs
    lookahead: bool = True          # put a turn on the device before the tokens of the turn before are read
    tile_rows: int = 128            # rows of a matrix-kernel tile: prompt portions make room for decode tokens (0: never)

    def __post_init__(self):
        for key in ("block_size", "kv_blocks", "max_context", "max_active", "max_queue",
                    "prefill_chunk", "min_prefill_chunk"):
            if getattr(self, key) <= 0:
                raise ValueError(f"{key} must be positive")
        if self.block_size % 4:
            raise ValueError("block_size must be a multiple of 4: the attention kernels read a page's keys four at a time")
        if self.prefill_chunk < self.min_prefill_chunk or self.target_step_ms <= 0:
            raise ValueError("invalid prefill control bounds")
        if self.dtype not in ("bfloat16", "float32"):
            raise ValueError("dtype must be bfloat16 or float32")
        if self.max_step_tokens < 0:
            raise ValueError("max_step_tokens must not be negative")
        if self.max_step_tokens and self.max_step_tokens < self.max_active + 1:
            raise ValueError("max_step_tokens must leave room for every decode token and one prompt token")

    @property
    def step_token_budget(self):
        return self.max_step_tokens or (self.max_active + self.prefill_chunk)

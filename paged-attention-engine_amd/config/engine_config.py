"""Settings of the engine that do not come from the model: cache and budgets.

Names follow the reference: BLOCK_SIZE, NUM_GPU_BLOCKS and
ADMISSION_MARGIN_BLOCKS are module constants there (engine/cache.py:29-35) and
`max_num_seqs`, `max_num_batched_tokens` and `admission_margin_blocks` are
keyword arguments of its Scheduler (engine/scheduler.py:317-349, None = unbounded).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

BLOCK_SIZE = 16
NUM_GPU_BLOCKS = 3584
ADMISSION_MARGIN_BLOCKS = 1

DTYPES = ("bfloat16", "float32")


@dataclass(frozen=True)
class EngineConfig:
    dtype: str = "bfloat16"
    block_size: int = BLOCK_SIZE
    num_blocks: int = NUM_GPU_BLOCKS
    admission_margin_blocks: int = ADMISSION_MARGIN_BLOCKS
    max_num_seqs: Optional[int] = None
    max_num_batched_tokens: Optional[int] = None
    num_state_slots: Optional[int] = None  # default: max_num_seqs, else 64
    device: str = "cuda:0"

    def __post_init__(self) -> None:
        if self.dtype not in DTYPES:
            raise ValueError(f"dtype must be one of {DTYPES}, got {self.dtype!r}")
        if self.block_size < 1:
            raise ValueError(f"block_size must be at least 1, got {self.block_size}")
        if self.num_blocks < 1:
            raise ValueError(f"num_blocks must be at least 1, got {self.num_blocks}")
        if self.admission_margin_blocks < 0:
            raise ValueError(
                f"admission_margin_blocks must be non-negative, got {self.admission_margin_blocks}")
        if self.max_num_seqs is not None and self.max_num_seqs < 1:
            raise ValueError(f"max_num_seqs must be at least 1, got {self.max_num_seqs}")
        if self.max_num_batched_tokens is not None and self.max_num_batched_tokens < 1:
            raise ValueError(
                f"max_num_batched_tokens must be at least 1, got {self.max_num_batched_tokens}")

    @property
    def state_slots(self) -> int:
        if self.num_state_slots is not None:
            return self.num_state_slots
        return self.max_num_seqs if self.max_num_seqs is not None else 64

"""Settings of the engine that do not come from the model: cache and budgets.

Names follow the reference: BLOCK_SIZE, NUM_GPU_BLOCKS and
ADMISSION_MARGIN_BLOCKS are module constants there (engine/cache.py:29-35) and
`max_num_seqs`, `max_num_batched_tokens` and `admission_margin_blocks` are
keyword arguments of its Scheduler (engine/scheduler.py:317-349, None = unbounded).
The reference's pool is a fixed number of pages (3,584, engine/cache.py:29-35;
bench/baseline.py:77-90 prices it in bytes); here the pool may also be given as a
byte budget (`kv_bytes`) or as a share of the device memory that is free once the
weights are in place (`fill_hbm`).
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
    num_blocks: Optional[int] = None      # pages per group; None with neither of the next two: NUM_GPU_BLOCKS
    kv_bytes: Optional[int] = None        # or: bytes the whole cache may take
    fill_hbm: Optional[float] = None      # or: this share (0..1] of the memory free after the weights
    admission_margin_blocks: int = ADMISSION_MARGIN_BLOCKS
    max_num_seqs: Optional[int] = None
    max_num_batched_tokens: Optional[int] = None
    num_state_slots: Optional[int] = None  # default: max_num_seqs; else see `state_slots_for`
    device: str = "cuda:0"

    def __post_init__(self) -> None:
        if self.dtype not in DTYPES:
            raise ValueError(f"dtype must be one of {DTYPES}, got {self.dtype!r}")
        if self.block_size < 1:
            raise ValueError(f"block_size must be at least 1, got {self.block_size}")
        given = [n for n in ("num_blocks", "kv_bytes", "fill_hbm") if getattr(self, n) is not None]
        if len(given) > 1:
            raise ValueError(f"the pool's size is given once: got {' and '.join(given)}")
        if self.num_blocks is not None and self.num_blocks < 1:
            raise ValueError(f"num_blocks must be at least 1, got {self.num_blocks}")
        if self.kv_bytes is not None and self.kv_bytes < 1:
            raise ValueError(f"kv_bytes must be positive, got {self.kv_bytes}")
        if self.fill_hbm is not None and not 0 < self.fill_hbm <= 1:
            raise ValueError(f"fill_hbm is a share of the free memory in (0, 1], got {self.fill_hbm}")
        if self.admission_margin_blocks < 0:
            raise ValueError(
                f"admission_margin_blocks must be non-negative, got {self.admission_margin_blocks}")
        if self.max_num_seqs is not None and self.max_num_seqs < 1:
            raise ValueError(f"max_num_seqs must be at least 1, got {self.max_num_seqs}")
        if self.max_num_batched_tokens is not None and self.max_num_batched_tokens < 1:
            raise ValueError(
                f"max_num_batched_tokens must be at least 1, got {self.max_num_batched_tokens}")

    def pages(self, page_bytes: int, free_bytes_now) -> int:
        """Pages per group: as given, or as many as the byte budget pays for at `page_bytes` for one
        page in every group.  `free_bytes_now()` is asked only for `fill_hbm`."""
        if self.kv_bytes is not None:
            count = self.kv_bytes // max(page_bytes, 1)
        elif self.fill_hbm is not None:
            count = int(free_bytes_now() * self.fill_hbm) // max(page_bytes, 1)
        else:
            return self.num_blocks if self.num_blocks is not None else NUM_GPU_BLOCKS
        if count < 1:
            raise ValueError(f"the cache's budget does not pay for one page of {page_bytes} bytes in every group")
        return count

    def state_slots_for(self, pages: int, keeps_state: bool) -> int:
        """Slots for per-request state, which also bound the live sequences: as given, else
        `max_num_seqs`.  With neither, a model that keeps no such state gets one slot per page (a live
        sequence holds at least a page, so the slots never bind); a model that does keep state has its
        slots allocated up front, and the caller must say how many."""
        if self.num_state_slots is not None:
            return self.num_state_slots
        if self.max_num_seqs is not None:
            return self.max_num_seqs
        if keeps_state:
            raise ValueError("this model keeps per-request state in slots that are allocated up front: "
                             "give max_num_seqs or num_state_slots")
        return max(1, pages)

"""Pages of one pool: a free list and the block table of every sequence.

Behaviour follows the reference's BlockAllocator (engine/cache.py:173-277): a
FIFO free list (pages are taken from the front and given back to the rear, so
reuse is as late as possible and a read of a freed page shows up as wrong data,
:180-184), all-or-nothing `append_tokens` that reports exhaustion as a value and
touches nothing (:238-257), KeyError for unknown or duplicate sequences, and the
invariant that every page is either free or in exactly one table.

Beyond the reference: `release_before`, which gives back the pages a window has
passed.  The table keeps a hole (-1) in their place so that logical block i
still covers positions [i * block_size, (i + 1) * block_size).
"""

from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from enum import Enum
from typing import Dict, List, Tuple

HOLE = -1


class AllocStatus(Enum):
    OK = "ok"
    OUT_OF_BLOCKS = "out_of_blocks"


@dataclass(frozen=True)
class AllocResult:
    status: AllocStatus
    new_block_ids: Tuple[int, ...] = ()

    @property
    def ok(self) -> bool:
        return self.status is AllocStatus.OK


@dataclass
class BlockTable:
    block_ids: List[int] = field(default_factory=list)
    num_tokens: int = 0
    released: int = 0  # leading logical blocks given back (holes)

    def __len__(self) -> int:
        return len(self.block_ids)

    @property
    def held(self) -> int:
        return len(self.block_ids) - self.released


class BlockAllocator:
    def __init__(self, num_blocks: int, block_size: int) -> None:
        if num_blocks < 1:
            raise ValueError(f"num_blocks must be at least 1, got {num_blocks}")
        if block_size < 1:
            raise ValueError(f"block_size must be at least 1, got {block_size}")
        self.num_blocks = num_blocks
        self.block_size = block_size
        self._free: deque = deque(range(num_blocks))
        self._tables: Dict[int, BlockTable] = {}

    # --- pool state
    @property
    def num_free(self) -> int:
        return len(self._free)

    @property
    def num_allocated(self) -> int:
        return sum(t.held for t in self._tables.values())

    def free_block_ids(self) -> Tuple[int, ...]:
        return tuple(self._free)

    def sequence_ids(self) -> Tuple[int, ...]:
        return tuple(self._tables)

    def blocks_needed(self, num_tokens: int) -> int:
        if num_tokens < 0:
            raise ValueError(f"num_tokens must be non-negative, got {num_tokens}")
        return -(-num_tokens // self.block_size)

    # --- per-sequence lifecycle
    def create_sequence(self, seq_id: int) -> None:
        if seq_id in self._tables:
            raise KeyError(f"sequence {seq_id} already exists")
        self._tables[seq_id] = BlockTable()

    def has_sequence(self, seq_id: int) -> bool:
        return seq_id in self._tables

    def block_table(self, seq_id: int) -> Tuple[int, ...]:
        return tuple(self._tables[seq_id].block_ids)

    def num_tokens(self, seq_id: int) -> int:
        return self._tables[seq_id].num_tokens

    def blocks_held(self, seq_id: int) -> int:
        return self._tables[seq_id].held

    def new_blocks_for(self, seq_id: int, count: int) -> int:
        """Pages `append_tokens(seq_id, count)` would take."""
        table = self._tables[seq_id]
        return self.blocks_needed(table.num_tokens + count) - len(table)

    def append_token(self, seq_id: int) -> AllocResult:
        return self.append_tokens(seq_id, 1)

    def append_tokens(self, seq_id: int, count: int) -> AllocResult:
        if count < 0:
            raise ValueError(f"count must be non-negative, got {count}")
        table = self._tables[seq_id]
        required = self.blocks_needed(table.num_tokens + count) - len(table)
        if required > len(self._free):
            return AllocResult(AllocStatus.OUT_OF_BLOCKS)
        taken = tuple(self._free.popleft() for _ in range(required))
        table.block_ids.extend(taken)
        table.num_tokens += count
        return AllocResult(AllocStatus.OK, new_block_ids=taken)

    def release_before(self, seq_id: int, position: int) -> Tuple[int, ...]:
        """Give back every page all of whose positions lie before `position`."""
        table = self._tables[seq_id]
        upto = min(max(position, 0) // self.block_size, len(table))
        freed = []
        for i in range(table.released, upto):
            freed.append(table.block_ids[i])
            table.block_ids[i] = HOLE
        table.released = max(table.released, upto)
        self._free.extend(freed)
        return tuple(freed)

    def free_sequence(self, seq_id: int) -> Tuple[int, ...]:
        table = self._tables.pop(seq_id)
        freed = tuple(b for b in table.block_ids if b != HOLE)
        self._free.extend(freed)
        return freed

    # --- address translation
    def physical_slot(self, seq_id: int, position: int) -> Tuple[int, int]:
        table = self._tables[seq_id]
        if not 0 <= position < table.num_tokens:
            raise IndexError(
                f"position {position} out of range for sequence {seq_id} holding {table.num_tokens} tokens")
        logical, offset = divmod(position, self.block_size)
        if table.block_ids[logical] == HOLE:
            raise IndexError(f"position {position} of sequence {seq_id} lies in a page already given back")
        return table.block_ids[logical], offset

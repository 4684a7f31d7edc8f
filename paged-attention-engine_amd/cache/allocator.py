"""Pages of one pool: who holds which, and in which order free pages go out.

What it does is what the reference's `BlockAllocator` does (engine/cache.py:173-277),
under the same method names, since those are the interface the reference's users know:

  * free pages go out oldest-first and come back to the rear (engine/cache.py:180-184:
    reuse as late as possible, so that reading a page after giving it back shows as
    wrong data rather than being hidden by getting the same page again);
  * `append_tokens` takes every page it needs or none, and says so with a value
    instead of raising (:238-257);
  * a page is free or held by exactly one sequence, and a sequence holds exactly the
    pages its token count needs (:176-178).

How it does it is this engine's own.  The free pages sit in a ring of fixed size (no
page is ever in it twice, so `num_blocks` cells are enough), every page carries its
holder's id so that `audit` can check the pool in one pass and a double return is
caught at the page, and a sequence's table is an `array('i')` that goes into the
step's staging buffer without conversion.  Beyond the reference, `release_before`
returns the leading pages that a sliding window has passed; their places in the table
become `HOLE`, so that table entry i still stands for positions
[i * block_size, (i + 1) * block_size).
"""

from __future__ import annotations

from array import array
from dataclasses import dataclass
from enum import Enum
from typing import Dict, Iterator, Tuple

HOLE = -1
_NOBODY = -1  # holder of a free page


class AllocStatus(Enum):
    OK = "ok"
    OUT_OF_BLOCKS = "out_of_blocks"


@dataclass(frozen=True)
class AllocResult:
    """What `append_tokens` did: the pages it took, or that the pool could not cover them."""

    status: AllocStatus
    new_block_ids: Tuple[int, ...] = ()

    @property
    def ok(self) -> bool:
        return self.status is AllocStatus.OK


_OUT_OF_BLOCKS = AllocResult(AllocStatus.OUT_OF_BLOCKS)


class BlockTable:
    """One sequence's pages in position order, with the count of its tokens and of the
    leading entries that are holes."""

    __slots__ = ("block_ids", "num_tokens", "released")

    def __init__(self) -> None:
        self.block_ids = array("i")
        self.num_tokens = 0
        self.released = 0

    def __len__(self) -> int:
        return len(self.block_ids)

    @property
    def held(self) -> int:
        return len(self.block_ids) - self.released


class _FreeRing:
    """First in, first out over page ids, in a ring of as many cells as there are pages."""

    __slots__ = ("_cells", "_head", "_count")

    def __init__(self, num_blocks: int) -> None:
        self._cells = array("i", range(num_blocks))
        self._head = 0
        self._count = num_blocks

    def __len__(self) -> int:
        return self._count

    def __iter__(self) -> Iterator[int]:
        size = len(self._cells)
        return (self._cells[(self._head + i) % size] for i in range(self._count))

    def take(self, n: int) -> Tuple[int, ...]:
        size = len(self._cells)
        out = tuple(self._cells[(self._head + i) % size] for i in range(n))
        self._head = (self._head + n) % size
        self._count -= n
        return out

    def give(self, page: int) -> None:
        size = len(self._cells)
        if self._count >= size:
            raise AssertionError("more pages returned than the pool has")
        self._cells[(self._head + self._count) % size] = page
        self._count += 1


class BlockAllocator:
    def __init__(self, num_blocks: int, block_size: int) -> None:
        for name, value in (("num_blocks", num_blocks), ("block_size", block_size)):
            if value < 1:
                raise ValueError(f"a pool needs {name} >= 1 (got {value})")
        self.num_blocks = num_blocks
        self.block_size = block_size
        self._ring = _FreeRing(num_blocks)
        self._holder = array("i", [_NOBODY]) * num_blocks
        self._tables: Dict[int, BlockTable] = {}
        self._held_total = 0

    # ------------------------------------------------------------------ the pool as a whole
    @property
    def num_free(self) -> int:
        return len(self._ring)

    @property
    def num_allocated(self) -> int:
        return self._held_total

    def free_block_ids(self) -> Tuple[int, ...]:
        """The free pages in the order they would go out."""
        return tuple(self._ring)

    def sequence_ids(self) -> Tuple[int, ...]:
        return tuple(self._tables)

    def blocks_needed(self, num_tokens: int) -> int:
        if num_tokens < 0:
            raise ValueError(f"a token count cannot be negative (got {num_tokens})")
        return (num_tokens + self.block_size - 1) // self.block_size

    def audit(self) -> None:
        """Check the pool against its invariants; AssertionError names the first breach."""
        seen = array("b", [0]) * self.num_blocks
        for page in self._ring:
            assert not seen[page], f"page {page} is in the free ring twice"
            assert self._holder[page] == _NOBODY, f"free page {page} is marked as held by {self._holder[page]}"
            seen[page] = 1
        held = 0
        for seq_id, table in self._tables.items():
            assert len(table) == self.blocks_needed(table.num_tokens), (
                f"sequence {seq_id}: {len(table)} table entries for {table.num_tokens} tokens")
            for index, page in enumerate(table.block_ids):
                if index < table.released:
                    assert page == HOLE, f"sequence {seq_id}: entry {index} was released but names page {page}"
                    continue
                assert page != HOLE, f"sequence {seq_id}: a hole at entry {index}, past the released ones"
                assert not seen[page], f"page {page} is held twice, or held and free"
                assert self._holder[page] == seq_id, f"page {page}: held by {seq_id}, marked {self._holder[page]}"
                seen[page] = 1
                held += 1
        assert held == self._held_total and held + len(self._ring) == self.num_blocks, (
            f"{held} held + {len(self._ring)} free pages of {self.num_blocks}")

    # ------------------------------------------------------------------ one sequence
    def _table(self, seq_id: int) -> BlockTable:
        try:
            return self._tables[seq_id]
        except KeyError:
            raise KeyError(f"the pool knows no sequence {seq_id}") from None

    def create_sequence(self, seq_id: int) -> None:
        if seq_id in self._tables:
            raise KeyError(f"sequence id {seq_id} is in use")
        self._tables[seq_id] = BlockTable()

    def has_sequence(self, seq_id: int) -> bool:
        return seq_id in self._tables

    def block_table(self, seq_id: int) -> Tuple[int, ...]:
        return tuple(self._table(seq_id).block_ids)

    def table_array(self, seq_id: int) -> array:
        """The table itself (not a copy), for the step's staging buffer: read, never written."""
        return self._table(seq_id).block_ids

    def num_tokens(self, seq_id: int) -> int:
        return self._table(seq_id).num_tokens

    def blocks_held(self, seq_id: int) -> int:
        return self._table(seq_id).held

    def new_blocks_for(self, seq_id: int, count: int) -> int:
        """How many pages `append_tokens(seq_id, count)` would take."""
        table = self._table(seq_id)
        return self.blocks_needed(table.num_tokens + count) - len(table)

    def append_token(self, seq_id: int) -> AllocResult:
        return self.append_tokens(seq_id, 1)

    def append_tokens(self, seq_id: int, count: int) -> AllocResult:
        if count < 0:
            raise ValueError(f"cannot append {count} tokens")
        table = self._table(seq_id)
        shortfall = self.blocks_needed(table.num_tokens + count) - len(table)
        if shortfall > len(self._ring):
            return _OUT_OF_BLOCKS  # nothing has been touched
        pages = self._ring.take(shortfall)
        for page in pages:
            self._holder[page] = seq_id
        table.block_ids.extend(pages)
        table.num_tokens += count
        self._held_total += shortfall
        return AllocResult(AllocStatus.OK, pages)

    def _give_back(self, seq_id: int, page: int) -> None:
        if self._holder[page] != seq_id:
            raise AssertionError(f"page {page} returned by sequence {seq_id}, which does not hold it")
        self._holder[page] = _NOBODY
        self._ring.give(page)
        self._held_total -= 1

    def release_before(self, seq_id: int, position: int) -> Tuple[int, ...]:
        """Return the pages that lie wholly before `position`; their table entries become holes."""
        table = self._table(seq_id)
        whole_pages = min(max(position, 0) // self.block_size, len(table))
        returned = []
        while table.released < whole_pages:
            page = table.block_ids[table.released]
            table.block_ids[table.released] = HOLE
            table.released += 1
            self._give_back(seq_id, page)
            returned.append(page)
        return tuple(returned)

    def free_sequence(self, seq_id: int) -> Tuple[int, ...]:
        """Forget the sequence; its pages come back in table order."""
        table = self._table(seq_id)
        del self._tables[seq_id]
        returned = tuple(table.block_ids[table.released:])
        for page in returned:
            self._give_back(seq_id, page)
        return returned

    # ------------------------------------------------------------------ where a token lives
    def physical_slot(self, seq_id: int, position: int) -> Tuple[int, int]:
        """(page, offset within the page) of the token at `position`."""
        table = self._table(seq_id)
        if position < 0 or position >= table.num_tokens:
            raise IndexError(f"sequence {seq_id} has tokens 0..{table.num_tokens - 1}; {position} is not one of them")
        entry, offset = divmod(position, self.block_size)
        if entry < table.released:
            raise IndexError(f"sequence {seq_id} has given back the page of position {position}")
        return table.block_ids[entry], offset

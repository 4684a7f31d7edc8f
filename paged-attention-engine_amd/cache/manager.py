"""The cache manager: paged keys and values in groups, and per-request state slots.

Each stop of the model's schedule declares what it keeps: per token (a
`PagedSpec`: key/value heads, head size and, if it only looks back a window,
that window) or per request (a `StateSpec` of fixed shape), or nothing.  Stops
with the same `PagedSpec` form a group: one pool of pages, one allocator and one
block table per sequence serve all of them, because they fill and pass pages in
lock step.  Groups with different needs have pools and tables of their own.

The reference has a single pool whose block ids index every layer's tensor
(engine/cache.py:305-341) and gives pages back only when a sequence finishes or
is evicted (engine/scheduler.py:614-645).  Here pages also return once a
window has passed them (`release_passed`).  A reservation takes pages in every
group or in none (the reference's all-or-nothing `append_tokens`,
engine/cache.py:238-257, carried over to several pools).

Pool layout of one group: [entry][K|V][block][kv head][block_size * head_dim]; the
keys of one (block, head) are one contiguous tile [block_size][head_dim], the
values one contiguous tile stored transposed, [head_dim][block_size], which is
what the attention kernels' matrix-core operands want.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Mapping, Optional, Sequence, Tuple

import torch

from .allocator import AllocResult, AllocStatus, BlockAllocator


@dataclass(frozen=True)
class PagedSpec:
    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclass(frozen=True)
class StateSpec:
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


class CacheGroup:
    def __init__(self, index: int, spec: PagedSpec, entries: List[int], num_blocks: int, block_size: int):
        self.index = index
        self.spec = spec
        self.entries = entries
        self.allocator = BlockAllocator(num_blocks, block_size)
        self.pool: Optional[torch.Tensor] = None

    def max_blocks_for(self, total_tokens: int, max_chunk: Optional[int]) -> int:
        """Most pages one sequence of `total_tokens` can hold at a time when it
        never runs more than `max_chunk` tokens in a step."""
        full = self.allocator.blocks_needed(total_tokens)
        if self.spec.window is None:
            return full
        chunk = total_tokens if max_chunk is None else min(max_chunk, total_tokens)
        return min(full, self.allocator.blocks_needed(self.spec.window - 1 + chunk) + 1)


class StateSlots:
    """Slots of fixed size for per-request state: taken when a sequence is
    created, given back when it is freed, FIFO like pages."""

    def __init__(self, num_slots: int) -> None:
        self.num_slots = num_slots
        self._free = list(range(num_slots))
        self._held: Dict[int, int] = {}

    @property
    def num_free(self) -> int:
        return len(self._free)

    def take(self, seq_id: int) -> Optional[int]:
        if seq_id in self._held:
            raise KeyError(f"sequence {seq_id} already holds a state slot")
        if not self._free:
            return None
        slot = self._free.pop(0)
        self._held[seq_id] = slot
        return slot

    def release(self, seq_id: int) -> int:
        slot = self._held.pop(seq_id)
        self._free.append(slot)
        return slot

    def slot_of(self, seq_id: int) -> int:
        return self._held[seq_id]

    def held(self) -> Mapping[int, int]:
        return dict(self._held)


class CacheManager:
    def __init__(self, paged: Sequence[Optional[PagedSpec]], states: Sequence[Optional[StateSpec]],
                 block_size: int, num_blocks, num_slots: int, dtype: torch.dtype = torch.float32,
                 device: Optional[str] = None) -> None:
        """`paged[i]` / `states[i]` describe schedule stop i (None: keeps nothing,
        or reads another stop's cache).  `num_blocks` is an int (every group gets
        that many pages) or a mapping from a group's window (None for full) to its count."""
        if len(paged) != len(states):
            raise ValueError("paged and states must describe the same stops")
        self.block_size = block_size
        self.dtype = dtype
        self.device = device
        self.groups: List[CacheGroup] = []
        self._group_of_entry: Dict[int, Tuple[int, int]] = {}  # entry -> (group, index within group)
        by_spec: Dict[PagedSpec, CacheGroup] = {}
        for entry, spec in enumerate(paged):
            if spec is None:
                continue
            if spec not in by_spec:
                count = num_blocks[spec.window] if isinstance(num_blocks, Mapping) else int(num_blocks)
                by_spec[spec] = CacheGroup(len(self.groups), spec, [], count, block_size)
                self.groups.append(by_spec[spec])
            group = by_spec[spec]
            self._group_of_entry[entry] = (group.index, len(group.entries))
            group.entries.append(entry)
        self.state_specs = list(states)
        self.slots = StateSlots(num_slots)
        self.state_tensors: Dict[int, torch.Tensor] = {}
        self._tokens: Dict[int, int] = {}
        if device is not None:
            for group in self.groups:
                s = group.spec
                group.pool = torch.zeros(
                    (len(group.entries), 2, group.allocator.num_blocks, s.num_kv_heads, block_size, s.head_dim),
                    dtype=dtype, device=device)
            for entry, spec in enumerate(states):
                if spec is not None:
                    self.state_tensors[entry] = torch.zeros((num_slots, *spec.shape), dtype=spec.dtype, device=device)

    # ------------------------------------------------------------------ lookups
    def group_of(self, entry: int) -> Optional[int]:
        hit = self._group_of_entry.get(entry)
        return None if hit is None else hit[0]

    def kv_of(self, entry: int) -> Tuple[torch.Tensor, torch.Tensor]:
        """(keys, values) pools of a stop: keys [block][kv head][block_size][head_dim],
        values [block][kv head][head_dim][block_size]."""
        g, i = self._group_of_entry[entry]
        pool = self.groups[g].pool
        return pool[i, 0], pool[i, 1].view(pool.shape[2], pool.shape[3], pool.shape[5], pool.shape[4])

    def state_of(self, entry: int) -> torch.Tensor:
        return self.state_tensors[entry]

    def storage_bytes(self) -> int:
        total = 0
        for group in self.groups:
            s = group.spec
            elem = torch.empty((), dtype=self.dtype).element_size()
            total += (len(group.entries) * 2 * group.allocator.num_blocks * s.num_kv_heads * self.block_size
                      * s.head_dim * elem)
        return total

    # ------------------------------------------------------------------ sequences
    def sequence_ids(self) -> Tuple[int, ...]:
        return tuple(self._tokens)

    def has_sequence(self, seq_id: int) -> bool:
        return seq_id in self._tokens

    def create_sequence(self, seq_id: int) -> bool:
        """Register an empty sequence and give it a state slot.  False (nothing
        changed) when no slot is free; KeyError when the id is already in use."""
        if seq_id in self._tokens:
            raise KeyError(f"sequence {seq_id} already exists")
        slot = self.slots.take(seq_id)
        if slot is None:
            return False
        for group in self.groups:
            group.allocator.create_sequence(seq_id)
        self._tokens[seq_id] = 0
        for tensor in self.state_tensors.values():
            tensor[slot].zero_()
        return True

    def num_tokens(self, seq_id: int) -> int:
        return self._tokens[seq_id]

    def slot_of(self, seq_id: int) -> int:
        return self.slots.slot_of(seq_id)

    def block_table(self, group: int, seq_id: int) -> Tuple[int, ...]:
        return self.groups[group].allocator.block_table(seq_id)

    def can_reserve(self, seq_id: int, count: int, margin: int = 0) -> bool:
        return all(g.allocator.new_blocks_for(seq_id, count) + margin <= g.allocator.num_free
                   for g in self.groups)

    def reserve(self, seq_id: int, count: int) -> AllocResult:
        """Room for `count` more tokens in every group, or in none."""
        if seq_id not in self._tokens:
            raise KeyError(f"unknown sequence {seq_id}")
        if not self.can_reserve(seq_id, count):
            return AllocResult(AllocStatus.OUT_OF_BLOCKS)
        taken: Tuple[int, ...] = ()
        for group in self.groups:
            result = group.allocator.append_tokens(seq_id, count)
            assert result.ok
            taken += result.new_block_ids
        self._tokens[seq_id] += count
        return AllocResult(AllocStatus.OK, taken)

    def release_passed(self, seq_id: int) -> int:
        """Give back the pages that no later token of `seq_id` can look at: in a
        group with window w, the next query (at position num_tokens) sees keys
        from num_tokens - w + 1 on.  Returns how many pages came back."""
        freed = 0
        n = self._tokens[seq_id]
        for group in self.groups:
            if group.spec.window is not None:
                freed += len(group.allocator.release_before(seq_id, n - group.spec.window + 1))
        return freed

    def free_sequence(self, seq_id: int) -> int:
        """Drop the sequence: every page and its state slot come back."""
        del self._tokens[seq_id]
        freed = 0
        for group in self.groups:
            freed += len(group.allocator.free_sequence(seq_id))
        self.slots.release(seq_id)
        return freed

    # ------------------------------------------------------------------ capacity arithmetic
    def fits_alone(self, total_tokens: int, margin: int, max_chunk: Optional[int] = None) -> bool:
        """Could a sequence that grows to `total_tokens` ever run, with `margin`
        pages kept aside in every group?  (The reference's admission guard,
        engine/scheduler.py:73-91.)"""
        return all(g.max_blocks_for(total_tokens, max_chunk) <= g.allocator.num_blocks - margin
                   for g in self.groups)

    def fits_now(self, total_tokens: int, margin: int, max_chunk: Optional[int] = None) -> bool:
        """Is there room now for a new sequence of `total_tokens`, leaving `margin`
        pages free in every group?  (engine/scheduler.py:376-379.)"""
        return self.slots.num_free > 0 and all(
            g.max_blocks_for(total_tokens, max_chunk) + margin <= g.allocator.num_free for g in self.groups)

    def free_blocks(self) -> Tuple[int, ...]:
        return tuple(g.allocator.num_free for g in self.groups)

    def min_free_blocks(self) -> int:
        return min((g.allocator.num_free for g in self.groups), default=0)

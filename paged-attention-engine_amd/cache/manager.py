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

What a page holds is the mixer's business: a `PagedSpec` lists named tensors, each
with the shape of one page of it, in which `PAGE` stands for the page's token count.
A group's pool is one tensor per name, [stop][block][*page shape].  The attention
mixer declares keys [kv head][PAGE][head_dim] (the keys of one (block, head) are one
contiguous tile) and values stored transposed, [kv head][head_dim][PAGE], which is
what its matrix-core kernels' operands want (`attention_pages`); a mixer that caches
one latent vector per token declares one tensor [PAGE][width], and the manager
needs no change for it.

Every pool has one page more than its allocator hands out, and the state tensors one
slot more (`padding_page`, `padding_slot`): rows that a recorded step is padded with
live there, where no sequence's data ever is.
"""

from __future__ import annotations

from dataclasses import dataclass
from collections import deque
from typing import Dict, List, Mapping, Optional, Sequence, Tuple, Union

import torch

from .allocator import AllocResult, AllocStatus, BlockAllocator

PAGE = "page"  # in a page shape: the number of tokens a page holds


@dataclass(frozen=True)
class PagedTensor:
    """One cached tensor: its name and the shape of one page of it (`PAGE` where the page's
    token count goes, which must appear exactly once)."""

    name: str
    page_shape: Tuple[Union[int, str], ...]

    def __post_init__(self) -> None:
        if sum(1 for d in self.page_shape if d == PAGE) != 1:
            raise ValueError(f"cached tensor '{self.name}': its page shape {self.page_shape} must name PAGE once")

    def shape(self, block_size: int) -> Tuple[int, ...]:
        return tuple(block_size if d == PAGE else int(d) for d in self.page_shape)

    def elements_per_token(self) -> int:
        count = 1
        for d in self.page_shape:
            count *= 1 if d == PAGE else int(d)
        return count


@dataclass(frozen=True)
class PagedSpec:
    """What a mixer keeps per token: named tensors and, if it only looks back so far, a window."""

    tensors: Tuple[PagedTensor, ...]
    window: Optional[int] = None

    def __post_init__(self) -> None:
        names = [t.name for t in self.tensors]
        if not names or len(set(names)) != len(names):
            raise ValueError(f"a paged spec needs tensors with distinct names, got {names}")

    def elements_per_token(self) -> int:
        return sum(t.elements_per_token() for t in self.tensors)


def attention_pages(num_kv_heads: int, head_dim: int, window: Optional[int] = None) -> PagedSpec:
    """Keys "k" [kv head][PAGE][head_dim] and values "v" [kv head][head_dim][PAGE] (transposed
    within the page), as the attention kernels read them."""
    return PagedSpec((PagedTensor("k", (num_kv_heads, PAGE, head_dim)),
                      PagedTensor("v", (num_kv_heads, head_dim, PAGE))), window)


@dataclass(frozen=True)
class StateSpec:
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


def bytes_of_one_page_everywhere(paged: Sequence[Optional[PagedSpec]], block_size: int, dtype: torch.dtype) -> int:
    """Bytes that one more page in every group's pool costs (all stops of all groups): what a
    pool of N pages per group takes is N times this."""
    elem = torch.empty((), dtype=dtype).element_size()
    return sum(spec.elements_per_token() for spec in paged if spec is not None) * block_size * elem


class CacheGroup:
    def __init__(self, index: int, spec: PagedSpec, entries: List[int], num_blocks: int, block_size: int):
        self.index = index
        self.spec = spec
        self.entries = entries
        self.allocator = BlockAllocator(num_blocks, block_size)
        self.pools: Dict[str, torch.Tensor] = {}  # tensor name -> [stop][block][*page shape]

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
        self._free = deque(range(num_slots))
        self._held: Dict[int, int] = {}

    @property
    def num_free(self) -> int:
        return len(self._free)

    def take(self, seq_id: int) -> Optional[int]:
        if seq_id in self._held:
            raise KeyError(f"sequence {seq_id} already holds a state slot")
        if not self._free:
            return None
        slot = self._free.popleft()
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
                for t in group.spec.tensors:
                    group.pools[t.name] = torch.zeros(
                        (len(group.entries), group.allocator.num_blocks + 1, *t.shape(block_size)),
                        dtype=dtype, device=device)
            for entry, spec in enumerate(states):
                if spec is not None:
                    self.state_tensors[entry] = torch.zeros((num_slots + 1, *spec.shape), dtype=spec.dtype,
                                                            device=device)

    # ------------------------------------------------------------------ lookups
    def padding_page(self, group: int) -> int:
        """The page of a group's pool that its allocator never hands out."""
        return self.groups[group].allocator.num_blocks

    @property
    def padding_slot(self) -> int:
        return self.slots.num_slots

    def group_of(self, entry: int) -> Optional[int]:
        hit = self._group_of_entry.get(entry)
        return None if hit is None else hit[0]

    def pages_of(self, entry: int) -> Dict[str, torch.Tensor]:
        """The cached tensors of a stop by name, each [block][*page shape]."""
        g, i = self._group_of_entry[entry]
        return {name: pool[i] for name, pool in self.groups[g].pools.items()}

    def state_of(self, entry: int) -> torch.Tensor:
        return self.state_tensors[entry]

    def storage_bytes(self) -> int:
        elem = torch.empty((), dtype=self.dtype).element_size()
        return sum(len(g.entries) * g.allocator.num_blocks * self.block_size * g.spec.elements_per_token() * elem
                   for g in self.groups)

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

    def table_array(self, group: int, seq_id: int):
        """The table itself as an array of int32, not a copy: for the step's staging buffer."""
        return self.groups[group].allocator.table_array(seq_id)

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

"""The step function: one batch of (sequence, its next tokens) through the model.

A step carries, for every sequence in it, the next tokens to run: a portion of a
prompt (any length, starting wherever the cache ends) or a single decoded token.
All of them run as one flat batch of T = sum of lengths rows, without padding,
from the cache that earlier steps left, and logits come back only for the rows
asked for.  The reference's counterpart is `forward_batch_prereserved`
(engine/model.py:408-455), which pads to a rectangle and returns the last row of
each sequence; like it, this function never allocates pages: the caller has
reserved room for every token (:414-417), so positions are the run
[tokens held before, tokens held now) (engine/attention.py:556-564).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from ..cache.manager import CacheManager
from ..parts import StepContext
from .model import Model


TILE_TOKENS = 32  # tokens per run handed to the prefill attention kernel


@dataclass(frozen=True)
class StepEntry:
    seq_id: int
    token_ids: Tuple[int, ...]
    want: Tuple[int, ...] = ()  # places among token_ids whose logits are returned


class StepRunner:
    def __init__(self, model: Model, cache: CacheManager) -> None:
        self.model = model
        self.cache = cache
        self.device = model.device
        self.vocab_size = model.plan.vocab_size

    def run(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        """Run one step.  Every entry's tokens must already be reserved in the
        cache (`cache.reserve(seq_id, len(token_ids))`), and they are the last
        tokens reserved.  Returns float32 logits [number of wanted places, vocab]
        in the order of the entries and of each entry's `want`."""
        cache = self.cache
        ids: List[int] = []
        positions: List[int] = []
        tok_seq: List[int] = []
        rows: List[int] = []
        seq_ids, q_starts, q_lens, past_lens, slots = [], [], [], [], []
        for row, entry in enumerate(entries):
            n = len(entry.token_ids)
            if n == 0:
                raise ValueError(f"sequence {entry.seq_id}: a step entry needs at least one token")
            held = cache.num_tokens(entry.seq_id)
            past = held - n
            if past < 0:
                raise ValueError(f"sequence {entry.seq_id}: {n} tokens to run but only {held} reserved")
            for tok in entry.token_ids:
                if not 0 <= tok < self.vocab_size:
                    raise ValueError(f"sequence {entry.seq_id}: token id {tok} outside the vocabulary "
                                     f"of {self.vocab_size}")
            for w in entry.want:
                if not 0 <= w < n:
                    raise ValueError(f"sequence {entry.seq_id}: wanted place {w} outside its {n} tokens")
                rows.append(len(ids) + w)
            seq_ids.append(entry.seq_id)
            q_starts.append(len(ids))
            q_lens.append(n)
            past_lens.append(past)
            slots.append(cache.slot_of(entry.seq_id))
            ids.extend(entry.token_ids)
            positions.extend(range(past, held))
            tok_seq.extend([row] * n)
        if len(set(seq_ids)) != len(seq_ids):
            raise ValueError("a sequence may appear only once in a step")
        if not ids:
            raise ValueError("a step needs at least one entry")

        # one staging buffer, one copy to the device
        T, S = len(ids), len(seq_ids)
        tables = []
        for group in cache.groups:
            per_seq = [cache.block_table(group.index, s) for s in seq_ids]
            width = max(1, max(len(t) for t in per_seq))
            tables.append((width, per_seq))
        decode_tokens = [q_starts[i] for i in range(S) if q_lens[i] == 1]
        tiles: List[int] = []
        for i in range(S):
            if q_lens[i] > 1:
                for first in range(0, q_lens[i], TILE_TOKENS):
                    tiles += [i, q_starts[i] + first, min(TILE_TOKENS, q_lens[i] - first)]
        total = 3 * T + S + len(rows) + len(decode_tokens) + len(tiles) + sum(S * w for w, _ in tables)
        staging = torch.empty(total, dtype=torch.int32, pin_memory=True)
        flat: List[int] = ids + positions + tok_seq + slots + rows + decode_tokens + tiles
        for width, per_seq in tables:
            for table in per_seq:
                flat.extend(table)
                flat.extend([-1] * (width - len(table)))
        staging.copy_(torch.tensor(flat, dtype=torch.int32))
        dev = staging.to(self.device, non_blocking=True)
        off = 0

        def take(count):
            nonlocal off
            out = dev[off:off + count]
            off += count
            return out

        d_ids, d_pos, d_seq, d_slots, d_rows = take(T), take(T), take(T), take(S), take(len(rows))
        d_decode, d_tiles = take(len(decode_tokens)), take(len(tiles)).view(-1, 3)
        block_tables: Dict[int, torch.Tensor] = {}
        for group, (width, _) in zip(cache.groups, tables):
            block_tables[group.index] = take(S * width).view(S, width)

        ctx = StepContext(dtype=self.model.dtype, device=self.device, num_tokens=T, num_seqs=S,
                          positions=d_pos, tok_seq=d_seq, block_tables=block_tables, slots=d_slots,
                          cache=cache, seq_ids=seq_ids, q_starts=q_starts, q_lens=q_lens,
                          past_lens=past_lens, host_slots=slots, decode_tokens=d_decode,
                          prefill_tiles=d_tiles)
        return self.model.forward(ctx, d_ids, d_rows)

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

import os
from array import array
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from ..cache.manager import CacheManager
from ..kernels import lib as K
from ..parts import StepContext, StepShape
from .model import Model


@dataclass(frozen=True)
class StepEntry:
    seq_id: int
    token_ids: Tuple[int, ...]
    want: Tuple[int, ...] = ()  # places among token_ids whose logits are returned


class _CapturedStep:
    """A decode step recorded as a HIP graph: static inputs, the graph, its logits."""

    def __init__(self, inputs: torch.Tensor, program=None) -> None:
        self.inputs = inputs
        self.program = program  # room for the step's layers as one resident kernel (made before the recording)
        self.graph: Optional[torch.cuda.CUDAGraph] = None
        self.logits: Optional[torch.Tensor] = None


def padded_rows(count: int) -> int:
    """Rows a recorded step of `count` sequences is padded to: every count up to 8, then multiples
    of 4 up to 32, then multiples of 8.  A stream whose batch shrinks and grows by one sequence
    at a time then replays a handful of recordings instead of making one per count."""
    if count <= 8:
        return count
    unit = 4 if count <= 32 else 8
    return -(-count // unit) * unit


class StepRunner:
    """Runs steps.  Steps in which every sequence brings exactly one token (decode
    steps) are recorded once per shape as a HIP graph and replayed, so that a step
    costs one copy of its inputs and one graph launch instead of hundreds of kernel
    launches; this needs every part of the model to be `graph_safe` (no host-side
    data in its forward) and is switched off otherwise.

    A recorded step is padded to `padded_rows` sequences.  A padding row is a sequence of its own
    that holds one token at position 0 in the cache's padding page and padding state slot (which
    no real sequence ever holds), so it reads and writes nothing that anyone looks at; its
    logits are dropped."""

    TABLE_ROUND = 64    # block tables of captured steps are padded to a multiple of this many pages
    MAX_GRAPHS = 24

    def __init__(self, model: Model, cache: CacheManager, use_graphs: bool = True,
                 use_programs: Optional[bool] = None) -> None:
        self.model = model
        self.cache = cache
        self.device = model.device
        self.vocab_size = model.plan.vocab_size
        self.use_graphs = use_graphs and model.graph_safe
        self.graph_max_rows = model.graph_max_rows
        self._list_parts = model.step_list_parts(cache.block_size)
        self._graphs: Dict[tuple, _CapturedStep] = {}
        self.graph_replays = 0
        self.graph_recordings = 0
        # Decode steps of a few rows can run their layers as one resident kernel where the model's parts
        # allow it (see kernels.lib.DecodeProgram): the same bits as the separate kernels.  It is off
        # unless asked for (`use_programs=True`, or PAE_DECODE_PROGRAMS=1): at the sizes measured the
        # barrier between its phases costs what a kernel boundary costs, and the step is slower.
        if use_programs is None:
            use_programs = os.environ.get("PAE_DECODE_PROGRAMS", "0") == "1"
        self.use_programs = bool(use_programs) and model.dtype == torch.bfloat16
        self.program_groups: Optional[int] = None  # workgroups of a program; None: one per compute unit
        self._eager_program = None
        self._programs: List = []
        # a slow check for tests and debugging: after every step, wait for the device and see that the
        # products' ticket counters are back at zero
        self.check_tickets = bool(os.environ.get("PAE_CHECK_TICKETS"))
        # pinned staging buffers that take turns, each with the event behind which the GPU has read it
        self._staging: List[Optional[torch.Tensor]] = [None] * self.STAGING_BUFFERS
        self._staging_read: List[Optional[torch.cuda.Event]] = [None] * self.STAGING_BUFFERS
        self._staging_turn = 0

    STAGING_BUFFERS = 4

    def _new_program(self):
        if not self.use_programs:
            return None
        program = K.DecodeProgram(self.device, self.model.max_program_phases(), self.program_groups)
        self._programs.append(program)
        return program

    def check_programs(self) -> None:
        """Raise if any decode program of this runner was abandoned at a barrier.  The device must
        have been waited for (a caller that holds the step's tokens has)."""
        for program in self._programs:
            program.check()

    def _to_device(self, flat: array, dst: Optional[torch.Tensor]) -> torch.Tensor:
        """A step's metadata to the device: into one of a few pinned buffers that take turns, and from
        there by a small kernel in line with the step's own kernels (no trip through the copy engine,
        no pinned allocation per step).  `dst`: the recorded step's input buffer, or None for a new one."""
        n = len(flat)
        turn = self._staging_turn
        self._staging_turn = (turn + 1) % self.STAGING_BUFFERS
        if self._staging_read[turn] is not None:
            self._staging_read[turn].synchronize()  # the step that used this buffer has read it (long ago)
        pinned = self._staging[turn]
        if pinned is None or pinned.numel() < n:
            pinned = self._staging[turn] = torch.empty(max(1024, 2 * n), dtype=torch.int32, pin_memory=True)
        pinned[:n].copy_(torch.frombuffer(flat, dtype=torch.int32))
        if dst is None:
            dst = torch.empty(n, dtype=torch.int32, device=self.device)
        K.copy_int32_from_pinned(dst, pinned, n)
        if self._staging_read[turn] is None:
            self._staging_read[turn] = torch.cuda.Event()
        self._staging_read[turn].record()
        return dst

    def run(self, entries: Sequence[StepEntry],
            feeds: Optional[Tuple[torch.Tensor, Sequence[Tuple[int, int]]]] = None) -> torch.Tensor:
        """Run one step.  Every entry's tokens must already be reserved in the
        cache (`cache.reserve(seq_id, len(token_ids))`), and they are the last
        tokens reserved.  Returns float32 logits [number of wanted places, vocab]
        in the order of the entries and of each entry's `want`.  The tensor may be
        overwritten by the next call.

        `feeds = (tokens, [(place, row), ...])`: token ids that are still on the device
        (an int32 tensor, the step before's samples): the flat token at `place` (counting
        through the entries) is `tokens[row]`, whatever the entry says there; at most one
        per sequence.  Nothing waits for the host to see those ids."""
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

        T, S, R = len(ids), len(seq_ids), len(rows)
        per_group = [[cache.table_array(group.index, s) for s in seq_ids] for group in cache.groups]
        decode_only = (self.use_graphs and T == S
                       and (self.graph_max_rows is None or padded_rows(S) <= self.graph_max_rows))
        if decode_only and padded_rows(S) > S:
            # padding rows: one token each at position 0 of a sequence that lives in the padding page
            extra = padded_rows(S) - S
            ids += [ids[0]] * extra
            positions += [0] * extra
            tok_seq += list(range(S, S + extra))
            q_starts += list(range(S, S + extra))
            q_lens += [1] * extra
            past_lens += [0] * extra
            slots += [cache.padding_slot] * extra
            seq_ids = seq_ids + [-1] * extra
            per_group = [tables + [array("i", [cache.padding_page(group.index)])] * extra
                         for group, tables in zip(cache.groups, per_group)]
            if R == S:  # every sequence samples: the padding rows' logits are computed and dropped
                rows += list(range(S, S + extra))
            T = S = S + extra
        widths = []
        for tables in per_group:
            width = max(1, max(len(t) for t in tables))
            if decode_only:
                width = -(-width // self.TABLE_ROUND) * self.TABLE_ROUND
            widths.append(width)

        # index lists that parts asked for (their kernels' work lists), built from the step's shape
        shape = StepShape(tuple(seq_ids), tuple(q_starts), tuple(q_lens), tuple(past_lens), cache.block_size)
        part_lists = [(key, name, list(flat), width) for key, part in self._list_parts.items()
                      for name, (flat, width) in part.step_lists(shape).items()]

        # one staging buffer, one copy to the device (see `_to_device`)
        # places and rows of token ids that come from the device, padded to one per sequence
        fed = list(feeds[1]) if feeds is not None else []
        if len(fed) > S or any(not (0 <= place < T and 0 <= row < feeds[0].numel()) for place, row in fed):
            raise ValueError("feeds: at most one per sequence, places within the step, rows within the tokens")
        fed_places = [place for place, _ in fed] + [0] * (S - len(fed))
        fed_rows = [row for _, row in fed] + [0] * (S - len(fed))
        flat = array("i", ids)
        for piece in (positions, tok_seq, slots, rows, fed_places, fed_rows):
            flat.extend(piece)
        list_offsets = []
        for _, _, values, _ in part_lists:
            flat.extend([0] * (-len(flat) % 4))  # every part's list starts on a 16-byte boundary
            list_offsets.append(len(flat))
            flat.extend(values)
        for width, tables in zip(widths, per_group):
            hole = array("i", [-1])
            for table in tables:
                flat.extend(table)
                flat.extend(hole * (width - len(table)))

        captured = None
        if decode_only:
            key = (S, len(rows), tuple(widths), tuple(len(values) for _, _, values, _ in part_lists))
            captured = self._graphs.pop(key, None)
            if captured is None:
                if len(self._graphs) >= self.MAX_GRAPHS:
                    # the recording that has gone unused the longest goes; a step launched from it
                    # may still be running
                    torch.cuda.current_stream().synchronize()
                    dropped = self._graphs.pop(next(iter(self._graphs)))
                    if dropped.program is not None:
                        dropped.program.check()
                        self._programs.remove(dropped.program)
                captured = _CapturedStep(torch.empty(len(flat), dtype=torch.int32, device=self.device),
                                         self._new_program())
            self._graphs[key] = captured  # last used, last to go
            dev = self._to_device(flat, captured.inputs)
        else:
            dev = self._to_device(flat, None)
        off = 0

        def take(count):
            nonlocal off
            out = dev[off:off + count]
            off += count
            return out

        d_ids, d_pos, d_seq, d_slots, d_rows = take(T), take(T), take(T), take(S), take(len(rows))
        d_fed_places, d_fed_rows = take(S), take(S)
        memo: Dict[object, object] = {}
        for (key, name, values, width), at in zip(part_lists, list_offsets):
            off = at
            tensor = take(len(values))
            memo.setdefault(key, {})[name] = tensor.view(-1, width) if width else tensor
        if fed:
            K.scatter_int32(d_ids, d_fed_places, feeds[0], d_fed_rows, len(fed))
        block_tables: Dict[int, torch.Tensor] = {}
        for group, width in zip(cache.groups, widths):
            block_tables[group.index] = take(S * width).view(S, width)

        program = None
        if self.use_programs and T == S:
            if captured is not None:
                program = captured.program
            else:  # a step launched kernel by kernel: one program serves them all, one after the other
                program = self._eager_program = self._eager_program or self._new_program()
        ctx = StepContext(dtype=self.model.dtype, device=self.device, num_tokens=T, num_seqs=S,
                          positions=d_pos, tok_seq=d_seq, block_tables=block_tables, slots=d_slots,
                          cache=cache, seq_ids=seq_ids, q_starts=q_starts, q_lens=q_lens,
                          past_lens=past_lens, host_slots=slots, memo=memo, program=program)
        if captured is None:
            logits = self.model.forward(ctx, d_ids, d_rows)
            if self.check_tickets:
                K.check_tickets_zero(self.device)
                self.check_programs()
            return logits
        if captured.graph is None:
            # record the step: nothing runs during the recording, so replay it right away
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                captured.logits = self.model.forward(ctx, d_ids, d_rows)
            captured.graph = graph
            self.graph_recordings += 1
        else:
            self.model.forward_pass_count += 1
        captured.graph.replay()
        self.graph_replays += 1
        if self.check_tickets:
            K.check_tickets_zero(self.device)
            self.check_programs()
        return captured.logits[:R]

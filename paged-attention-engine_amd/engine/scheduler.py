"""Continuous batching over the page pool: admit, cut prompts into portions, decode, finish.

Names, events and policies follow the reference's scheduler (engine/scheduler.py):

  * `Request(request_id, prompt_token_ids, max_new_tokens)` with a non-empty prompt
    and at least one new token (:148-167); EOS is ignored unless stop tokens are
    given, so exactly `max_new_tokens` are produced (engine/model.py:466-469).
  * The admission guard: a request whose full length could never fit in
    `num_blocks - admission_margin_blocks` pages is rejected at `add_request`
    and never queued (:73-91,423-449).
  * Strict first-come-first-served admission without backfilling (:496-518);
    preempted sequences re-enter by arrival order (:641-645).
  * Admission needs room for the whole current history plus the margin
    (:376-379); growth may spend the margin (:381-385).
  * When a sequence cannot grow, the newest running sequences are evicted until
    it can, or until it is itself the victim (:647-674); a victim loses its pages
    and its planned work, keeps what it generated, and replays prompt plus
    generated tokens when readmitted (:520-552,624-645).
  * `run_to_completion(max_steps)` raises when no progress is made (:753-770).

Different from the reference, whose step pads a rectangle and always prefills a
whole history in one step: the token budget `max_num_batched_tokens` counts real
tokens; running sequences decode first (one token each; a decode that the
budget refuses is deferred, keeps its pages and runs next step, as in :717-725),
then half-done prompts continue, then the queue's head is admitted, and any
prompt or replay longer than what is left of the budget runs in portions over
several steps.  A portion that contains the history's last token yields the next
token in that same step.  The reference's escape "an empty batch admits the head
whatever its length" (:484-494) becomes "an empty batch always runs at least
one token".  Every step is one call of the executor: one pass of the model.
"""

from __future__ import annotations

import time
from collections import deque
from dataclasses import dataclass, field
from enum import Enum
from typing import Callable, Dict, List, Optional, Protocol, Sequence as TypingSequence, Tuple

from ..cache.manager import CacheManager
from ..config.engine_config import ADMISSION_MARGIN_BLOCKS


# A generated token whose value is still on the device (see `Scheduler.run_overlapped`).
PENDING = -1


class EventKind(Enum):
    ADMIT = "admit"
    FINISH = "finish"
    PREEMPT = "preempt"
    RECOMPUTE = "recompute"
    REJECT = "reject"


@dataclass(frozen=True)
class Event:
    timestamp: float
    step: int
    kind: EventKind
    request_id: str
    detail: str
    free_blocks: int
    running: int
    waiting: int
    tokens_held: int = 0


@dataclass(frozen=True)
class Request:
    request_id: str
    prompt_token_ids: Tuple[int, ...]
    max_new_tokens: int
    temperature: float = 0.0
    seed: int = 0
    stop_token_ids: Tuple[int, ...] = ()

    def __post_init__(self) -> None:
        object.__setattr__(self, "prompt_token_ids", tuple(int(t) for t in self.prompt_token_ids))
        object.__setattr__(self, "stop_token_ids", tuple(int(t) for t in self.stop_token_ids))
        if not self.prompt_token_ids:
            raise ValueError(f"{self.request_id}: prompt must be non-empty")
        if self.max_new_tokens < 1:
            raise ValueError(f"{self.request_id}: max_new_tokens must be at least 1")
        if self.temperature < 0:
            raise ValueError(f"{self.request_id}: temperature must be non-negative")

    @property
    def prompt_len(self) -> int:
        return len(self.prompt_token_ids)

    @property
    def max_total_len(self) -> int:
        return self.prompt_len + self.max_new_tokens


class SequenceStatus(Enum):
    WAITING = "waiting"
    RUNNING = "running"
    FINISHED = "finished"
    REJECTED = "rejected"


@dataclass
class Sequence:
    """Runtime state of one request; survives preemption and readmission."""

    request: Request
    arrival_index: int
    generated: List[int] = field(default_factory=list)
    status: SequenceStatus = SequenceStatus.WAITING
    seq_id: Optional[int] = None
    num_computed: int = 0          # tokens of the history whose keys and values are cached
    prefilling: bool = False       # admitted, and the history's last token has not run yet
    preemption_count: int = 0      # telemetry only; never consulted by a decision
    step_logits: list = field(default_factory=list)  # with record_logits: one row per generated token
    stopped: bool = False

    @property
    def request_id(self) -> str:
        return self.request.request_id

    @property
    def history(self) -> List[int]:
        return list(self.request.prompt_token_ids) + self.generated

    @property
    def history_len(self) -> int:
        return self.request.prompt_len + len(self.generated)

    def history_slice(self, start: int, end: int) -> Tuple[int, ...]:
        """history[start:end] without building the whole history (a decode step asks for one token)."""
        prompt = self.request.prompt_token_ids
        n = len(prompt)
        if start >= n:
            return tuple(self.generated[start - n:end - n])
        if end <= n:
            return tuple(prompt[start:end])
        return tuple(prompt[start:]) + tuple(self.generated[:end - n])

    @property
    def is_finished(self) -> bool:
        return self.stopped or len(self.generated) >= self.request.max_new_tokens


@dataclass(frozen=True)
class ScheduledWork:
    """One sequence's share of a step: tokens, where they stand, and whether the
    last of them is the history's last (then its logits give the next token)."""

    seq: Sequence
    token_ids: Tuple[int, ...]
    positions: Tuple[int, ...]
    is_prefill: bool
    samples: bool


@dataclass(frozen=True)
class StepResult:
    step: int
    admitted: Tuple[str, ...]
    decoded: Tuple[str, ...]
    finished: Tuple[str, ...]
    preempted: Tuple[str, ...]
    running: int
    waiting: int
    free_blocks: int
    batch_size: int = 0
    deferred: Tuple[str, ...] = ()
    batched_token_cost: int = 0     # real tokens the step ran
    prefilled: Tuple[str, ...] = ()  # sequences that ran a prompt portion


class Executor(Protocol):
    """What the scheduler needs of a model: run one step's work in one pass and
    return, for every item that `samples`, its next token (None for the others)."""

    def execute(self, work: TypingSequence[ScheduledWork], record_logits: bool = False): ...


def is_admissible(max_total_len: int, cache: CacheManager,
                  admission_margin_blocks: int = ADMISSION_MARGIN_BLOCKS,
                  max_chunk: Optional[int] = None) -> bool:
    """The admission guard as a predicate (reference: engine/scheduler.py:78-91)."""
    return cache.fits_alone(max_total_len, admission_margin_blocks, max_chunk)


class Scheduler:
    def __init__(self, executor: Executor, cache: CacheManager,
                 admission_margin_blocks: int = ADMISSION_MARGIN_BLOCKS,
                 clock: Callable[[], float] = time.monotonic, record_logits: bool = False,
                 max_num_seqs: Optional[int] = None, max_num_batched_tokens: Optional[int] = None,
                 max_positions: Optional[int] = None) -> None:
        if admission_margin_blocks < 0:
            raise ValueError(f"admission_margin_blocks must be non-negative, got {admission_margin_blocks}")
        if max_num_seqs is not None and max_num_seqs < 1:
            raise ValueError(f"max_num_seqs must be at least 1, got {max_num_seqs}")
        if max_num_batched_tokens is not None and max_num_batched_tokens < 1:
            raise ValueError(f"max_num_batched_tokens must be at least 1, got {max_num_batched_tokens}")
        self.executor = executor
        self.cache = cache
        self.admission_margin_blocks = admission_margin_blocks
        self.clock = clock
        self.record_logits = record_logits
        self.max_num_seqs = max_num_seqs
        self.max_num_batched_tokens = max_num_batched_tokens
        self.max_positions = max_positions

        self.waiting: deque = deque()
        self.running: List[Sequence] = []
        self.finished: Dict[str, Sequence] = {}
        self.rejected: Dict[str, Sequence] = {}
        self.events: List[Event] = []

        self._step = 0
        self._next_arrival = 0
        self._next_seq_id = 0
        self._pending: List[ScheduledWork] = []
        self._pending_tokens = 0

    # ------------------------------------------------------------------ event log
    def _tokens_held(self) -> int:
        return sum(self.cache.num_tokens(s.seq_id) for s in self.running if s.seq_id is not None)

    def _log(self, kind: EventKind, seq: Sequence, detail: str = "") -> None:
        self.events.append(Event(self.clock(), self._step, kind, seq.request_id, detail,
                                 self.cache.min_free_blocks(), len(self.running), len(self.waiting),
                                 self._tokens_held()))

    def events_of(self, kind: EventKind) -> List[Event]:
        return [e for e in self.events if e.kind is kind]

    # ------------------------------------------------------------------ intake
    def add_request(self, request: Request) -> bool:
        """Offer a request; False if it is rejected (it could never fit, or it is
        longer than the model's positions)."""
        seq = Sequence(request=request, arrival_index=self._next_arrival)
        self._next_arrival += 1
        reason = None
        if not is_admissible(request.max_total_len, self.cache, self.admission_margin_blocks,
                             self.max_num_batched_tokens):
            reason = (f"max length {request.max_total_len} cannot fit the pool with "
                      f"{self.admission_margin_blocks} page(s) kept aside "
                      f"(pages per group: {[g.allocator.num_blocks for g in self.cache.groups]})")
        elif self.max_positions is not None and request.max_total_len > self.max_positions:
            reason = f"max length {request.max_total_len} exceeds the model's {self.max_positions} positions"
        if reason is not None:
            seq.status = SequenceStatus.REJECTED
            self.rejected[request.request_id] = seq
            self._log(EventKind.REJECT, seq, reason)
            return False
        self.waiting.append(seq)
        return True

    # ------------------------------------------------------------------ budget
    def _tokens_planned(self) -> int:
        return self._pending_tokens  # kept beside `_pending` by `_plan`, `_evict` and `step`

    def _budget_left(self) -> int:
        """Tokens this step may still take; an empty batch may always take one."""
        if self.max_num_batched_tokens is None:
            return 1 << 60
        return max(self.max_num_batched_tokens - self._tokens_planned(), 0 if self._pending else 1)

    # ------------------------------------------------------------------ planning
    def _plan(self, seq: Sequence, count: int) -> None:
        """Reserve room for and queue the next `count` tokens of `seq`'s history."""
        result = self.cache.reserve(seq.seq_id, count)
        if not result.ok:
            raise AssertionError(f"{seq.request_id}: reserving {count} token(s) failed after the capacity check")
        start = seq.num_computed
        end = start + count
        self._pending.append(ScheduledWork(
            seq=seq, token_ids=seq.history_slice(start, end), positions=tuple(range(start, end)),
            is_prefill=seq.prefilling, samples=end == seq.history_len))
        self._pending_tokens += count

    def _evict(self, seq: Sequence) -> None:
        self.running.remove(seq)
        self._pending = [w for w in self._pending if w.seq is not seq]
        self._pending_tokens = sum(len(w.token_ids) for w in self._pending)
        freed = self.cache.free_sequence(seq.seq_id)
        seq.seq_id = None
        seq.num_computed = 0
        seq.prefilling = False
        seq.status = SequenceStatus.WAITING
        seq.preemption_count += 1
        self._log(EventKind.PREEMPT, seq, f"freed {freed} blocks, {len(seq.generated)} generated tokens to replay")
        self.waiting.append(seq)
        self.waiting = deque(sorted(self.waiting, key=lambda s: s.arrival_index))

    def _make_room_for(self, seq: Sequence, count: int) -> List[Sequence]:
        """Evict newest-first until `seq` can take `count` more tokens, or until it
        is itself the victim.  The victims are never the whole running set: the
        admission guard bounds every sequence to what the pool holds alone."""
        running_before = len(self.running)
        victims: List[Sequence] = []
        while not self.cache.can_reserve(seq.seq_id, count):
            if not self.running:
                raise AssertionError(f"{seq.request_id}: nothing left to evict but still cannot allocate")
            victim = max(self.running, key=lambda s: s.arrival_index)
            victims.append(victim)
            self._evict(victim)
            if victim is seq:
                break
        assert len(victims) < running_before, (
            f"eviction victim set ({len(victims)}) is the entire running set ({running_before})")
        return victims

    def _start(self, seq: Sequence) -> None:
        is_recompute = bool(seq.generated)
        seq.seq_id = self._next_seq_id
        self._next_seq_id += 1
        if not self.cache.create_sequence(seq.seq_id):
            raise AssertionError(f"{seq.request_id}: no state slot after the capacity check")
        seq.status = SequenceStatus.RUNNING
        seq.num_computed = 0
        seq.prefilling = True
        self.running.append(seq)
        self._log(EventKind.ADMIT, seq, f"prefill {seq.history_len} tokens"
                  + (f", readmission #{seq.preemption_count}" if is_recompute else ""))
        if is_recompute:
            self._log(EventKind.RECOMPUTE, seq,
                      f"replaying {seq.history_len} tokens ({seq.request.prompt_len} prompt + "
                      f"{len(seq.generated)} generated)")

    def _finish(self, seq: Sequence) -> None:
        self.running.remove(seq)
        freed = self.cache.free_sequence(seq.seq_id)
        seq.seq_id = None
        seq.status = SequenceStatus.FINISHED
        self.finished[seq.request_id] = seq
        self._log(EventKind.FINISH, seq, f"{len(seq.generated)} tokens, freed {freed} blocks")

    # ------------------------------------------------------------------ the step
    def _plan_batch(self):
        """Decide a step: what runs, who is evicted, who is admitted.  Pages are reserved and
        the work is queued; nothing has run yet."""
        self._step += 1
        self._pending = []
        self._pending_tokens = 0
        preempted: List[str] = []
        deferred: List[str] = []
        admitted: List[Sequence] = []

        # 1. sequences already running, in running order: decodes and prompt portions
        for want_prefill in (False, True):
            for seq in list(self.running):
                if seq.status is not SequenceStatus.RUNNING:
                    continue  # evicted earlier in this step
                remaining = seq.history_len - seq.num_computed
                if seq.prefilling != want_prefill:
                    continue
                count = min(remaining, self._budget_left())
                if count < 1:
                    deferred.append(seq.request_id)
                    continue
                if not self.cache.can_reserve(seq.seq_id, count):
                    victims = self._make_room_for(seq, count)
                    preempted.extend(v.request_id for v in victims)
                    if seq.status is not SequenceStatus.RUNNING:
                        continue  # it was its own victim
                self._plan(seq, count)

        # 2. admission from the head of the queue: strict arrival order, no backfilling;
        #    a step that had to evict admits nobody (the pages it freed are spoken for)
        while self.waiting and not preempted:
            head = self.waiting[0]
            if self.max_num_seqs is not None and len(self.running) >= self.max_num_seqs:
                break
            if not self.cache.fits_now(head.history_len, self.admission_margin_blocks,
                                       self.max_num_batched_tokens):
                break
            budget = self._budget_left()
            if budget < 1:
                break
            self.waiting.popleft()
            self._start(head)
            admitted.append(head)
            self._plan(head, min(head.history_len, budget))

        batch = self._pending
        self._pending = []
        tokens_run, self._pending_tokens = self._pending_tokens, 0
        return batch, tokens_run, preempted, deferred, admitted

    def _advance(self, work: ScheduledWork, token: Optional[int], row=None) -> None:
        """What a work item that has run (or is sure to) changes: the sequence's progress, the
        pages a window has passed, and for an item that samples its new token (PENDING while
        the value is still on the device), a stop, the end."""
        seq = work.seq
        seq.num_computed += len(work.token_ids)
        self.cache.release_passed(seq.seq_id)
        if not work.samples:
            return
        if token is None:
            raise AssertionError(f"{seq.request_id}: executor returned no token for a sampling item")
        seq.prefilling = False
        if self.record_logits:
            seq.step_logits.append(row)
        seq.generated.append(int(token))
        if int(token) in seq.request.stop_token_ids:
            seq.stopped = True
        if seq.is_finished:
            self._finish(seq)

    def _result(self, batch, tokens_run, preempted, deferred, admitted, finished_before) -> StepResult:
        return StepResult(
            step=self._step,
            admitted=tuple(s.request_id for s in admitted),
            decoded=tuple(w.seq.request_id for w in batch if not w.is_prefill),
            finished=tuple(sorted(set(self.finished) - finished_before)),
            preempted=tuple(preempted),
            running=len(self.running),
            waiting=len(self.waiting),
            free_blocks=self.cache.min_free_blocks(),
            batch_size=len(batch),
            deferred=tuple(deferred),
            batched_token_cost=tokens_run,
            prefilled=tuple(w.seq.request_id for w in batch if w.is_prefill),
        )

    def step(self) -> StepResult:
        finished_before = set(self.finished)
        batch, tokens_run, preempted, deferred, admitted = self._plan_batch()
        # one pass of the model for everything planned
        if batch:
            results = self.executor.execute(batch, self.record_logits)
            if len(results) != len(batch):
                raise AssertionError(f"executor returned {len(results)} results for {len(batch)} items")
            for work, result in zip(batch, results):
                token, row = result if isinstance(result, tuple) else (result, None)
                self._advance(work, token if work.samples else None, row)
        return self._result(batch, tokens_run, preempted, deferred, admitted, finished_before)

    # ------------------------------------------------------------------ steps that overlap
    def can_overlap(self) -> bool:
        """Whether `run_overlapped` may be used: the executor can launch without waiting, no
        logits are recorded, and no request stops on a token's value."""
        every = list(self.waiting) + list(self.running)
        return (hasattr(self.executor, "launch") and not self.record_logits
                and not any(s.request.stop_token_ids for s in every))

    def run_overlapped(self, max_steps: int = 100_000, until_idle: bool = True) -> int:
        """Steps of which the next is decided and launched while the current one runs.

        What a step decides depends on the step before only through counts (who has how many
        tokens, who ends at `max_new_tokens`, which pages are free), never through a token's
        value, as long as no request has stop tokens: so after a step is launched its sequences
        are advanced with PENDING in place of their new tokens, the next step is planned and
        launched (the device hands the sampled ids over: `executor.launch`), and only then the
        host waits for the earlier step's tokens and writes them over the PENDINGs.  Decisions,
        events and tokens are those of `step()` called in a loop; the GPU does not wait for
        the host between steps.  Runs until nothing is left (or `max_steps` steps, with
        `until_idle=False`); returns the number of steps."""
        if not self.can_overlap():
            raise RuntimeError("run_overlapped needs an executor with launch(), no recorded logits and no stop tokens")
        steps = 0
        in_flight = None  # (launched step, its sampling work items)
        while (self.waiting or self.running) and steps < max_steps:
            batch, _, _, _, _ = self._plan_batch()
            steps += 1
            launched = self.executor.launch(batch, in_flight) if batch else None
            for work in batch:
                self._advance(work, PENDING if work.samples else None)
            if in_flight is not None:
                self._settle(in_flight)
            in_flight = launched
            if not batch and in_flight is None and until_idle:
                raise RuntimeError(f"no progress: {len(self.waiting)} waiting, {len(self.running)} running")
        if in_flight is not None:
            self._settle(in_flight)
        if until_idle and (self.waiting or self.running):
            raise RuntimeError(f"no progress after {max_steps} steps: {len(self.waiting)} waiting, "
                               f"{len(self.running)} running")
        return steps

    def _settle(self, launched) -> None:
        """The tokens of a launched step have arrived: write them where PENDING stands."""
        tokens = launched.wait()
        for work, token in zip(launched.sampling, tokens):
            seq = work.seq
            at = work.positions[-1] + 1 - seq.request.prompt_len  # index of this item's token among the generated
            if seq.generated[at] != PENDING:
                raise AssertionError(f"{seq.request_id}: token {at} was settled twice")
            seq.generated[at] = int(token)

    def run_to_completion(self, max_steps: int = 100_000) -> Dict[str, Tuple[int, ...]]:
        steps = 0
        while self.waiting or self.running:
            self.step()
            steps += 1
            if steps > max_steps:
                raise RuntimeError(f"no progress after {max_steps} steps: {len(self.waiting)} waiting, "
                                   f"{len(self.running)} running")
        return {rid: tuple(seq.generated) for rid, seq in self.finished.items()}

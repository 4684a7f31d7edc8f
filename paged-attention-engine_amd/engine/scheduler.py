"""Continuous batching over the page pool: admit, cut prompts into portions, decode, finish.

The policies are the reference scheduler's (engine/scheduler.py), and so are the names
its users see (`Request`, `add_request`, `step`, `run_to_completion`, the event kinds,
the fields of `StepResult`):

  * a request has a non-empty prompt and at least one new token to make (:148-167);
    an end-of-sequence token is ignored unless stop tokens are given, so exactly
    `max_new_tokens` come out (engine/model.py:466-469);
  * a request whose full length could never fit in the pool less the admission
    margin is turned away at `add_request` and never queued (:73-91,423-449);
  * admission is strictly in arrival order and nothing overtakes a head that does
    not fit (:496-518); a preempted request goes back to its place by arrival (:641-645);
  * admission needs room for the whole current history plus the margin (:376-379);
    growth may spend the margin (:381-385);
  * when a sequence cannot grow, the newest running sequences lose their pages until
    it can, or until it is itself the one that goes (:647-674); such a sequence keeps
    what it generated and replays prompt plus generated tokens when it comes back
    (:520-552,624-645);
  * `run_to_completion(max_steps)` raises when the work does not end (:753-770).

What differs comes from the step function.  The reference pads a rectangle and
prefills a whole history at once; here `max_num_batched_tokens` counts real tokens,
running sequences decode first (one token each; one that the budget refuses waits a
step with its pages, as in :717-725), half-done prompts go on next, the head of the
queue is admitted last, and a prompt or replay longer than what the budget leaves runs
in portions over several steps.  The portion that holds the history's last token gives
the next token in the same step.  Where the reference lets an empty batch admit the
head whatever its length (:484-494), an empty batch here may always run one token.
A step is one call of the executor, which is one pass of the model.
"""

from __future__ import annotations

import bisect
import time
from dataclasses import dataclass
from enum import Enum
from typing import Callable, Dict, Iterator, List, Optional, Protocol, Sequence as TypingSequence, Tuple

from ..cache.manager import CacheManager
from ..config.engine_config import ADMISSION_MARGIN_BLOCKS

# A generated token whose value is still on the device (see `Scheduler.run_overlapped`).
PENDING = -1
_NO_LIMIT = 1 << 60


class EventKind(Enum):
    ADMIT = "admit"
    FINISH = "finish"
    PREEMPT = "preempt"
    RECOMPUTE = "recompute"
    REJECT = "reject"


@dataclass(frozen=True)
class Event:
    """A decision and the pool as it stood then: free pages (capacity) and tokens held (occupancy)."""

    timestamp: float
    step: int
    kind: EventKind
    request_id: str
    detail: str
    free_blocks: int
    running: int
    waiting: int
    tokens_held: int = 0


def _as_ids(values, what: str, owner: str) -> Tuple[int, ...]:
    try:
        return tuple(int(v) for v in values)
    except (TypeError, ValueError):
        raise ValueError(f"request {owner}: {what} must be integers") from None


@dataclass(frozen=True)
class Request:
    request_id: str
    prompt_token_ids: Tuple[int, ...]
    max_new_tokens: int
    temperature: float = 0.0
    seed: int = 0
    stop_token_ids: Tuple[int, ...] = ()

    def __post_init__(self) -> None:
        rid = self.request_id
        object.__setattr__(self, "prompt_token_ids", _as_ids(self.prompt_token_ids, "prompt token ids", rid))
        object.__setattr__(self, "stop_token_ids", _as_ids(self.stop_token_ids, "stop token ids", rid))
        problems = []
        if len(self.prompt_token_ids) == 0:
            problems.append("an empty prompt")
        if self.max_new_tokens < 1:
            problems.append(f"max_new_tokens = {self.max_new_tokens} (at least 1 is needed)")
        if self.temperature < 0:
            problems.append(f"a negative temperature ({self.temperature})")
        if problems:
            raise ValueError(f"request {rid} has " + " and ".join(problems))

    @property
    def prompt_len(self) -> int:
        return len(self.prompt_token_ids)

    @property
    def max_total_len(self) -> int:
        return len(self.prompt_token_ids) + self.max_new_tokens


class SequenceStatus(Enum):
    WAITING = "waiting"
    RUNNING = "running"
    FINISHED = "finished"
    REJECTED = "rejected"


class Sequence:
    """A request on its way through the scheduler.  One object lives from `add_request` to
    the end, through any number of preemptions: `generated` only ever grows."""

    __slots__ = ("request", "arrival_index", "generated", "status", "seq_id", "num_computed", "prefilling",
                 "preemption_count", "step_logits", "stopped")

    def __init__(self, request: Request, arrival_index: int) -> None:
        self.request = request
        self.arrival_index = arrival_index      # place in the queue, first time and every time after
        self.generated: List[int] = []
        self.status = SequenceStatus.WAITING
        self.seq_id: Optional[int] = None       # its name in the cache while it holds pages
        self.num_computed = 0                   # tokens of the history whose keys and values are cached
        self.prefilling = False                 # admitted, and the history's last token has not run yet
        self.preemption_count = 0               # for the record; no decision reads it
        self.step_logits: list = []             # with record_logits: the row that gave each generated token
        self.stopped = False                    # a stop token came out

    def __repr__(self) -> str:
        return (f"Sequence({self.request.request_id!r}, {self.status.value}, "
                f"{self.num_computed}/{self.history_len} cached, {len(self.generated)} generated)")

    @property
    def request_id(self) -> str:
        return self.request.request_id

    @property
    def history_len(self) -> int:
        return len(self.request.prompt_token_ids) + len(self.generated)

    @property
    def history(self) -> List[int]:
        return [*self.request.prompt_token_ids, *self.generated]

    def history_slice(self, start: int, end: int) -> Tuple[int, ...]:
        """Tokens start..end-1 of prompt + generated, without joining the two for one decoded token."""
        prompt = self.request.prompt_token_ids
        split = len(prompt)
        head = prompt[start:end] if start < split else ()
        tail = self.generated[max(start, split) - split:end - split] if end > split else ()
        return (*head, *tail)

    @property
    def is_finished(self) -> bool:
        return self.stopped or len(self.generated) >= self.request.max_new_tokens


class ArrivalQueue:
    """Waiting sequences in arrival order; a preempted one slots back in by its arrival."""

    def __init__(self) -> None:
        self._order: List[int] = []
        self._seqs: List[Sequence] = []

    def __len__(self) -> int:
        return len(self._seqs)

    def __iter__(self) -> Iterator[Sequence]:
        return iter(self._seqs)

    def __getitem__(self, index):
        return self._seqs[index]

    def put(self, seq: Sequence) -> None:
        at = bisect.bisect_left(self._order, seq.arrival_index)
        self._order.insert(at, seq.arrival_index)
        self._seqs.insert(at, seq)

    def head(self) -> Sequence:
        return self._seqs[0]

    def take_head(self) -> Sequence:
        del self._order[0]
        return self._seqs.pop(0)


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


class _Plan:
    """A step while it is being decided."""

    __slots__ = ("work", "tokens", "preempted", "deferred", "admitted")

    def __init__(self) -> None:
        self.work: List[ScheduledWork] = []
        self.tokens = 0
        self.preempted: List[str] = []
        self.deferred: List[str] = []
        self.admitted: List[Sequence] = []

    def add(self, item: ScheduledWork) -> None:
        self.work.append(item)
        self.tokens += len(item.token_ids)

    def drop(self, seq: Sequence) -> None:
        kept = [w for w in self.work if w.seq is not seq]
        self.tokens -= sum(len(w.token_ids) for w in self.work) - sum(len(w.token_ids) for w in kept)
        self.work = kept


class Scheduler:
    def __init__(self, executor: Executor, cache: CacheManager,
                 admission_margin_blocks: int = ADMISSION_MARGIN_BLOCKS,
                 clock: Callable[[], float] = time.monotonic, record_logits: bool = False,
                 max_num_seqs: Optional[int] = None, max_num_batched_tokens: Optional[int] = None,
                 max_positions: Optional[int] = None) -> None:
        if admission_margin_blocks < 0:
            raise ValueError(f"admission_margin_blocks = {admission_margin_blocks}: pages cannot be kept aside in the negative")
        for name, value in (("max_num_seqs", max_num_seqs), ("max_num_batched_tokens", max_num_batched_tokens)):
            if value is not None and value < 1:
                raise ValueError(f"{name} = {value}: give None for no limit, or at least 1")
        self.executor = executor
        self.cache = cache
        self.admission_margin_blocks = admission_margin_blocks
        self.clock = clock
        self.record_logits = record_logits
        self.max_num_seqs = max_num_seqs
        self.max_num_batched_tokens = max_num_batched_tokens
        self.max_positions = max_positions

        self.waiting = ArrivalQueue()
        self.running: List[Sequence] = []
        self.finished: Dict[str, Sequence] = {}
        self.rejected: Dict[str, Sequence] = {}
        self.events: List[Event] = []

        self._step = 0
        self._arrivals = 0
        self._cache_ids = 0
        self._plan: Optional[_Plan] = None

    # ------------------------------------------------------------------ event log
    def _note(self, kind: EventKind, seq: Sequence, detail: str = "") -> None:
        held = sum(self.cache.num_tokens(s.seq_id) for s in self.running if s.seq_id is not None)
        self.events.append(Event(self.clock(), self._step, kind, seq.request_id, detail,
                                 self.cache.min_free_blocks(), len(self.running), len(self.waiting), held))

    def events_of(self, kind: EventKind) -> List[Event]:
        return [e for e in self.events if e.kind is kind]

    @property
    def idle(self) -> bool:
        return not self.running and not len(self.waiting)

    # ------------------------------------------------------------------ intake
    def _why_never(self, request: Request) -> Optional[str]:
        """Why this request could not run even alone, or None."""
        need = request.max_total_len
        if not is_admissible(need, self.cache, self.admission_margin_blocks, self.max_num_batched_tokens):
            pools = ", ".join(str(g.allocator.num_blocks) for g in self.cache.groups)
            return (f"max length {need} cannot fit: {self.cache.block_size}-token pages, {pools} per group, "
                    f"{self.admission_margin_blocks} kept aside")
        if self.max_positions is not None and need > self.max_positions:
            return f"max length {need} exceeds the model's {self.max_positions} positions"
        return None

    def add_request(self, request: Request) -> bool:
        """Queue a request.  False: it was turned away for good (see the REJECT event's detail)."""
        seq = Sequence(request, self._arrivals)
        self._arrivals += 1
        refusal = self._why_never(request)
        if refusal is None:
            self.waiting.put(seq)
            return True
        seq.status = SequenceStatus.REJECTED
        self.rejected[request.request_id] = seq
        self._note(EventKind.REJECT, seq, refusal)
        return False

    # ------------------------------------------------------------------ building a step
    def _budget_left(self) -> int:
        """Tokens the step being decided may still take; an empty one may always take one."""
        if self.max_num_batched_tokens is None:
            return _NO_LIMIT
        left = self.max_num_batched_tokens - self._plan.tokens
        return max(left, 0) if self._plan.work else max(left, 1)

    def _queue_tokens(self, seq: Sequence, count: int) -> None:
        """Take pages for the next `count` tokens of `seq`'s history and put them into the step."""
        if not self.cache.reserve(seq.seq_id, count).ok:
            raise AssertionError(f"{seq.request_id}: the pool refused {count} token(s) it had room for a moment ago")
        first, after = seq.num_computed, seq.num_computed + count
        self._plan.add(ScheduledWork(seq, seq.history_slice(first, after), tuple(range(first, after)),
                                     is_prefill=seq.prefilling, samples=after == seq.history_len))

    def _preempt(self, victim: Sequence) -> None:
        """Take a running sequence's pages and send it back to the queue."""
        self.running.remove(victim)
        if self._plan is not None:
            self._plan.drop(victim)  # what it was to run this step would read pages it no longer has
        pages = self.cache.free_sequence(victim.seq_id)
        victim.seq_id = None
        victim.num_computed = 0
        victim.prefilling = False
        victim.status = SequenceStatus.WAITING
        victim.preemption_count += 1
        self._note(EventKind.PREEMPT, victim,
                   f"gave back {pages} pages; {victim.history_len} tokens to replay, {len(victim.generated)} of them generated")
        self.waiting.put(victim)

    def _free_pages_for(self, seq: Sequence, count: int) -> List[Sequence]:
        """Preempt running sequences, newest arrival first, until `seq` has room for `count` more
        tokens or has gone itself.  The admission guard sizes every request to fit the pool alone,
        so there is always somebody left running afterwards."""
        were_running = len(self.running)
        gone: List[Sequence] = []
        for victim in sorted(self.running, key=lambda s: s.arrival_index, reverse=True):
            if self.cache.can_reserve(seq.seq_id, count):
                break
            self._preempt(victim)
            gone.append(victim)
            if victim is seq:
                break
        else:
            if not self.cache.can_reserve(seq.seq_id, count):
                raise AssertionError(f"{seq.request_id}: every sequence was preempted and {count} token(s) still "
                                     "do not fit; the admission guard lets no such request in")
        if len(gone) >= were_running:
            raise AssertionError(f"all {were_running} running sequences were preempted in one step; "
                                 "the admission guard lets no request in that needs this")
        return gone

    def _admit(self, seq: Sequence) -> None:
        replay = len(seq.generated) > 0
        seq.seq_id, self._cache_ids = self._cache_ids, self._cache_ids + 1
        if not self.cache.create_sequence(seq.seq_id):
            raise AssertionError(f"{seq.request_id}: admitted without a free state slot")
        seq.status = SequenceStatus.RUNNING
        seq.num_computed = 0
        seq.prefilling = True
        self.running.append(seq)
        self._plan.admitted.append(seq)
        self._note(EventKind.ADMIT, seq, f"prefill {seq.history_len} tokens"
                   + (f", readmission #{seq.preemption_count}" if replay else ""))
        if replay:
            self._note(EventKind.RECOMPUTE, seq, f"replaying {seq.history_len} tokens: "
                       f"{seq.request.prompt_len} of the prompt, {len(seq.generated)} generated")

    def _retire(self, seq: Sequence) -> None:
        self.running.remove(seq)
        pages = self.cache.free_sequence(seq.seq_id)
        seq.seq_id = None
        seq.status = SequenceStatus.FINISHED
        self.finished[seq.request_id] = seq
        self._note(EventKind.FINISH, seq, f"{len(seq.generated)} tokens, freed {pages} blocks")

    def _continue_running(self, prefilling: bool) -> None:
        """Give every running sequence of one kind (decoding, or still in its prompt) its next tokens."""
        plan = self._plan
        for seq in tuple(self.running):
            if seq.status is not SequenceStatus.RUNNING or seq.prefilling != prefilling:
                continue  # preempted a moment ago, or the other kind
            count = min(seq.history_len - seq.num_computed, self._budget_left())
            if count < 1:
                plan.deferred.append(seq.request_id)  # keeps its pages, runs next step
                continue
            if not self.cache.can_reserve(seq.seq_id, count):
                plan.preempted += [v.request_id for v in self._free_pages_for(seq, count)]
                if seq.status is not SequenceStatus.RUNNING:
                    continue  # it was the last to go
            self._queue_tokens(seq, count)

    def _admit_from_queue(self) -> None:
        """The queue's head, and the next, and so on while each fits: arrival order, no overtaking."""
        while len(self.waiting):
            if self.max_num_seqs is not None and len(self.running) >= self.max_num_seqs:
                return
            head = self.waiting.head()
            if not self.cache.fits_now(head.history_len, self.admission_margin_blocks, self.max_num_batched_tokens):
                return
            room = self._budget_left()
            if room < 1:
                return
            self._admit(self.waiting.take_head())
            self._queue_tokens(head, min(head.history_len, room))

    def _plan_batch(self) -> _Plan:
        """Decide a step: what runs, who is preempted, who is admitted.  Pages are taken and the work
        is listed; nothing has run yet."""
        self._step += 1
        plan = self._plan = _Plan()
        self._continue_running(prefilling=False)  # decodes first
        self._continue_running(prefilling=True)   # then prompts under way
        if not plan.preempted:
            # a step that had to preempt admits nobody: the pages it freed are spoken for
            self._admit_from_queue()
        self._plan = None
        return plan

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
            raise AssertionError(f"{seq.request_id}: the executor gave no token for an item that samples")
        token = int(token)
        seq.prefilling = False
        if self.record_logits:
            seq.step_logits.append(row)
        seq.generated.append(token)
        seq.stopped = token in seq.request.stop_token_ids
        if seq.is_finished:
            self._retire(seq)

    def _result(self, plan: _Plan, finished_before) -> StepResult:
        return StepResult(
            step=self._step,
            admitted=tuple(s.request_id for s in plan.admitted),
            decoded=tuple(w.seq.request_id for w in plan.work if not w.is_prefill),
            finished=tuple(sorted(set(self.finished) - finished_before)),
            preempted=tuple(plan.preempted),
            running=len(self.running),
            waiting=len(self.waiting),
            free_blocks=self.cache.min_free_blocks(),
            batch_size=len(plan.work),
            deferred=tuple(plan.deferred),
            batched_token_cost=plan.tokens,
            prefilled=tuple(w.seq.request_id for w in plan.work if w.is_prefill),
        )

    def step(self) -> StepResult:
        finished_before = set(self.finished)
        plan = self._plan_batch()
        if plan.work:  # one pass of the model for everything planned
            results = self.executor.execute(plan.work, self.record_logits)
            if len(results) != len(plan.work):
                raise AssertionError(f"{len(plan.work)} work items went to the executor, {len(results)} results came back")
            for work, result in zip(plan.work, results):
                token, row = result if isinstance(result, tuple) else (result, None)
                self._advance(work, token if work.samples else None, row)
        return self._result(plan, finished_before)

    # ------------------------------------------------------------------ steps that overlap
    def can_overlap(self) -> bool:
        """Whether `run_overlapped` may be used: the executor can launch without waiting, no
        logits are recorded, and no request stops on a token's value."""
        if self.record_logits or not hasattr(self.executor, "launch"):
            return False
        return not any(s.request.stop_token_ids for s in (*self.waiting, *self.running))

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
        in_flight = None  # the step launched last, not yet waited for
        while not self.idle and steps < max_steps:
            plan = self._plan_batch()
            steps += 1
            launched = self.executor.launch(plan.work, in_flight) if plan.work else None
            for work in plan.work:
                self._advance(work, PENDING if work.samples else None)
            if in_flight is not None:
                self._settle(in_flight)
            in_flight = launched
            if launched is None and until_idle:
                raise RuntimeError(f"a step ran nothing with {len(self.waiting)} waiting and {len(self.running)} running")
        if in_flight is not None:
            self._settle(in_flight)
        if until_idle and not self.idle:
            raise RuntimeError(f"{max_steps} steps did not finish the work: {len(self.waiting)} waiting, "
                               f"{len(self.running)} running")
        return steps

    def _settle(self, launched) -> None:
        """The tokens of a launched step have arrived: write them where PENDING stands."""
        for work, token in zip(launched.sampling, launched.wait()):
            seq = work.seq
            at = work.positions[-1] + 1 - seq.request.prompt_len  # which generated token this item made
            if seq.generated[at] != PENDING:
                raise AssertionError(f"{seq.request_id}: generated token {at} arrived twice")
            seq.generated[at] = int(token)

    def run_to_completion(self, max_steps: int = 100_000) -> Dict[str, Tuple[int, ...]]:
        """Step until nothing waits or runs; {request id: generated tokens}.  `max_steps` only
        catches a scheduler that has stopped getting anywhere."""
        for _ in range(max_steps + 1):
            if self.idle:
                return {rid: tuple(seq.generated) for rid, seq in self.finished.items()}
            self.step()
        raise RuntimeError(f"{max_steps} steps did not finish the work: {len(self.waiting)} waiting, "
                           f"{len(self.running)} running")

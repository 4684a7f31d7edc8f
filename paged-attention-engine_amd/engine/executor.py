"""The executor the scheduler drives: one step's work through the step function,
then sampling.  Counterpart of the reference's Qwen2Executor
(engine/scheduler.py:275-298), with the cache's bookkeeping left to the scheduler."""

from __future__ import annotations

from typing import Dict, List, Optional, Sequence

from ..cache.manager import CacheManager
from ..sampling import Sampler, uniform_for
from ..sampling.sampler import SampledTokens
from .model import Model
from .scheduler import PENDING
from .step import StepEntry, StepRunner


class LaunchedStep:
    """A step that has been handed to the GPU: its tokens, and which row is whose."""

    def __init__(self, tokens: SampledTokens, row_of: Dict[int, int], sampling: List, runner=None) -> None:
        self.tokens = tokens
        self.row_of = row_of      # id(sequence) -> row of its token
        self.sampling = sampling  # the work items that sample, in row order
        self.runner = runner

    def wait(self) -> List[int]:
        tokens = self.tokens.wait()
        if self.runner is not None:
            self.runner.check_programs()  # the step has finished: did its resident kernel get through?
        return tokens


class ModelExecutor:
    def __init__(self, model: Model, cache: CacheManager) -> None:
        self.model = model
        self.cache = cache
        self.runner = StepRunner(model, cache)
        self.sampler = Sampler(model.device)

    @staticmethod
    def _uniforms(sampling: Sequence) -> List[float]:
        """The draw of every item that samples with a temperature (greedy items need none)."""
        return [uniform_for(w.seq.request.seed, w.seq.request_id, len(w.seq.generated))
                if w.seq.request.temperature > 0 else 0.0 for w in sampling]

    def execute(self, work: Sequence, record_logits: bool = False) -> List:
        entries = [StepEntry(w.seq.seq_id, w.token_ids, (len(w.token_ids) - 1,) if w.samples else ())
                   for w in work]
        logits = self.runner.run(entries)
        sampling = [w for w in work if w.samples]
        temperatures = [w.seq.request.temperature for w in sampling]
        uniforms = self._uniforms(sampling)
        tokens = self.sampler.sample(logits, temperatures, uniforms)
        self.runner.check_programs()  # the tokens are on the host, so the step has finished
        rows = logits.cpu() if record_logits else None
        out, k = [], 0
        for w in work:
            if not w.samples:
                out.append(None)
                continue
            out.append((tokens[k], rows[k].clone()) if record_logits else tokens[k])
            k += 1
        return out

    def launch(self, work: Sequence, previous: Optional[LaunchedStep] = None) -> LaunchedStep:
        """Hand a step to the GPU and return without waiting for its tokens.  A token id that
        reads PENDING is the one `previous` sampled for that sequence: it is taken from
        `previous`'s tokens on the device."""
        entries, pairs, place = [], [], 0
        for w in work:
            ids = tuple(w.token_ids)
            if PENDING in ids:
                at = ids.index(PENDING)
                if previous is None or id(w.seq) not in previous.row_of or PENDING in ids[at + 1:]:
                    raise AssertionError(f"{w.seq.request_id}: a pending token without the step that samples it")
                pairs.append((place + at, previous.row_of[id(w.seq)]))
                ids = ids[:at] + (0,) + ids[at + 1:]
            entries.append(StepEntry(w.seq.seq_id, ids, (len(ids) - 1,) if w.samples else ()))
            place += len(ids)
        logits = self.runner.run(entries, (previous.tokens.on_device, pairs) if pairs else None)
        sampling = [w for w in work if w.samples]
        temperatures = [w.seq.request.temperature for w in sampling]
        uniforms = self._uniforms(sampling)
        tokens = self.sampler.sample_on_device(logits, temperatures, uniforms)
        return LaunchedStep(tokens, {id(w.seq): k for k, w in enumerate(sampling)}, sampling, self.runner)

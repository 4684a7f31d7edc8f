"""The executor the scheduler drives: one step's work through the step function,
then sampling.  Counterpart of the reference's Qwen2Executor
(engine/scheduler.py:275-298), with the cache's bookkeeping left to the scheduler."""

from __future__ import annotations

from typing import List, Sequence

from ..cache.manager import CacheManager
from ..sampling import Sampler, uniform_for
from .model import Model
from .step import StepEntry, StepRunner


class ModelExecutor:
    def __init__(self, model: Model, cache: CacheManager) -> None:
        self.model = model
        self.cache = cache
        self.runner = StepRunner(model, cache)
        self.sampler = Sampler(model.device)

    def execute(self, work: Sequence, record_logits: bool = False) -> List:
        entries = [StepEntry(w.seq.seq_id, w.token_ids, (len(w.token_ids) - 1,) if w.samples else ())
                   for w in work]
        logits = self.runner.run(entries)
        sampling = [w for w in work if w.samples]
        temperatures = [w.seq.request.temperature for w in sampling]
        uniforms = [uniform_for(w.seq.request.seed, w.seq.request_id, len(w.seq.generated)) for w in sampling]
        tokens = self.sampler.sample(logits, temperatures, uniforms)
        rows = logits.cpu() if record_logits else None
        out, k = [], 0
        for w in work:
            if not w.samples:
                out.append(None)
                continue
            out.append((tokens[k], rows[k].clone()) if record_logits else tokens[k])
            k += 1
        return out

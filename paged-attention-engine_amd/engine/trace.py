"""Trace replay: given token ids, step by step, through the engine's own model,
step function, cache and kernels, writing the logits asked for.  It samples nothing.

The reference has no such program; its nearest pieces are `record_logits`
(engine/scheduler.py:192-197,607-609) and the test helpers that build
(past, new) batches by hand (tests/test_fused.py:380-400).
"""

from __future__ import annotations

import json
import os
import sys
from typing import Dict, IO

import numpy as np

from ..config.engine_config import BLOCK_SIZE
from .model import TORCH_DTYPE, load_model
from .step import StepEntry, StepRunner

ROUND_TO = 64  # a request's token count is rounded up to this when the pool is sized


class TraceReplayer:
    def __init__(self, model, dtype: str, max_tokens: int, block_size: int = BLOCK_SIZE,
                 max_live: int = 4, device: str = "cuda:0") -> None:
        """`model`: a model folder, or a `Model` that is already built (then `dtype` must be its own)."""
        if ROUND_TO % block_size:
            raise ValueError(f"block_size {block_size} must divide {ROUND_TO}")
        self.model = load_model(model, dtype, device) if isinstance(model, str) else model
        if self.model.dtype != TORCH_DTYPE[dtype]:
            raise ValueError(f"replay in {dtype} asked of a model that computes in {self.model.dtype}")
        num_blocks = max(1, -(-max_tokens // ROUND_TO) * (ROUND_TO // block_size))
        self.cache = self.model.new_cache(block_size, num_blocks, max_live)
        self.runner = StepRunner(self.model, self.cache)
        self._seq_of: Dict[str, int] = {}
        self._next_seq = 0

    def step(self, record: dict):
        """Run one step record; returns float32 logits [wanted, vocab] or None."""
        entries = []
        for item in record.get("entries", []):
            rid = str(item["id"])
            tokens = tuple(int(t) for t in item["tokens"])
            if rid not in self._seq_of:
                seq_id = self._next_seq
                self._next_seq += 1
                if not self.cache.create_sequence(seq_id):
                    raise RuntimeError(f"request {rid}: more live requests than state slots")
                self._seq_of[rid] = seq_id
            seq_id = self._seq_of[rid]
            if not self.cache.reserve(seq_id, len(tokens)).ok:
                raise RuntimeError(f"request {rid}: the page pool is exhausted "
                                   f"(free pages per group: {self.cache.free_blocks()})")
            entries.append(StepEntry(seq_id, tokens, tuple(int(w) for w in item.get("want", []))))
        logits = None
        if entries:
            out = self.runner.run(entries)
            if out.shape[0]:
                logits = out.cpu().numpy()
                self.runner.check_programs()
            for entry in entries:
                self.cache.release_passed(entry.seq_id)
        for rid in record.get("end", []):
            self.cache.free_sequence(self._seq_of.pop(str(rid)))
        return logits


def replay(model_dir: str, dtype: str, out_dir: str, max_tokens: int, stream: IO[str],
           block_size: int = BLOCK_SIZE, report: IO[str] = sys.stdout) -> int:
    os.makedirs(out_dir, exist_ok=True)
    replayer = TraceReplayer(model_dir, dtype, max_tokens, block_size)
    for line in stream:
        line = line.strip()
        if not line:
            continue
        record = json.loads(line)
        logits = replayer.step(record)
        if logits is not None:
            np.ascontiguousarray(logits, dtype="<f4").tofile(os.path.join(out_dir, f"{record['step']}.f32"))
        print(f"done {record['step']}", file=report, flush=True)
    return 0

"""The Python entry point: a model folder in, generated token ids out.

The reference's README composes the same pieces by hand (README.md:27-44):
`Qwen2Engine.from_hf_model`, `BlockAllocator(num_blocks, block_size)`,
`engine.new_paged_cache(...)`, `Scheduler(Qwen2Executor(...), allocator,
max_num_seqs=64, max_num_batched_tokens=8192)`, `add_request(Request("r0",
prompt_token_ids=(1, 2, 3), max_new_tokens=32))`, `run_to_completion()` giving
`{request_id: (token, ...)}`.  `Engine` does that composition for a folder and
keeps the same method names; `generate` mirrors `generate_greedy`
(engine/model.py:459-503), returning tokens and the logits that produced them.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple, Union

import torch

from ..config.engine_config import ADMISSION_MARGIN_BLOCKS, BLOCK_SIZE, EngineConfig
from .executor import ModelExecutor
from .model import NAME_OF_DTYPE, TORCH_DTYPE, Model, load_model, random_model
from .scheduler import EventKind, Request, Scheduler, StepResult


@dataclass(frozen=True)
class GenerationResult:
    """`step_logits[i]` is the float32 row that produced `token_ids[i]`."""

    token_ids: Tuple[int, ...]
    step_logits: Optional[torch.Tensor]


class Engine:
    def __init__(self, model: Union[str, Model], dtype: Optional[str] = None, block_size: int = BLOCK_SIZE,
                 num_blocks: Optional[int] = None, max_num_seqs: Optional[int] = None,
                 max_num_batched_tokens: Optional[int] = None,
                 admission_margin_blocks: int = ADMISSION_MARGIN_BLOCKS, record_logits: bool = False,
                 device: str = "cuda:0", kv_bytes: Optional[int] = None, fill_hbm: Optional[float] = None,
                 num_state_slots: Optional[int] = None) -> None:
        """`model`: a folder, or a built `Model`.  `dtype`: "bfloat16" or "float32"; None takes the
        folder's own (`torch_dtype` of its config.json), or the built model's.  The pool: `num_blocks`
        pages in every cache group (default 3,584), or `kv_bytes` for the whole cache, or `fill_hbm`,
        the share of the device memory still free once the weights are in place."""
        if isinstance(model, str):
            model = load_model(model, dtype, device)
        if dtype is None:
            dtype = NAME_OF_DTYPE[model.dtype]
        self.config = EngineConfig(dtype=dtype, block_size=block_size, num_blocks=num_blocks, kv_bytes=kv_bytes,
                                   fill_hbm=fill_hbm, admission_margin_blocks=admission_margin_blocks,
                                   max_num_seqs=max_num_seqs, max_num_batched_tokens=max_num_batched_tokens,
                                   num_state_slots=num_state_slots, device=device)
        self.model = model
        if self.model.dtype != TORCH_DTYPE[dtype]:
            raise ValueError(f"the engine was asked for {dtype} but the model it was given computes in {self.model.dtype}")
        self.num_blocks = self.config.pages(self.model.page_bytes(block_size), self._free_device_bytes)
        keeps_state = any(spec is not None for spec in self.model.cache_specs()[1])
        self.cache = self.model.new_cache(block_size, self.num_blocks,
                                          self.config.state_slots_for(self.num_blocks, keeps_state))
        self.executor = ModelExecutor(self.model, self.cache)
        self.record_logits = record_logits
        self.scheduler = self._new_scheduler()

    @classmethod
    def from_random(cls, config, seed: int = 0, dtype: Optional[str] = None, device: str = "cuda:0",
                    std: float = 0.02, norm_std: float = 0.0, **engine_options) -> "Engine":
        """An engine over random weights drawn on the device from `seed` (no folder is written);
        `config` is a config.json dict or a typed config."""
        return cls(random_model(config, seed, dtype, device, std, norm_std), dtype=dtype, device=device,
                   **engine_options)

    def _free_device_bytes(self) -> int:
        torch.cuda.empty_cache()
        return torch.cuda.mem_get_info(torch.device(self.config.device))[0]

    def _new_scheduler(self) -> Scheduler:
        c = self.config
        return Scheduler(self.executor, self.cache, admission_margin_blocks=c.admission_margin_blocks,
                         record_logits=self.record_logits, max_num_seqs=c.max_num_seqs,
                         max_num_batched_tokens=c.max_num_batched_tokens,
                         max_positions=self.model.plan.max_positions)

    # the reference's scheduler surface
    def add_request(self, request: Union[Request, str], prompt_token_ids: Sequence[int] = (),
                    max_new_tokens: int = 1, temperature: float = 0.0, seed: int = 0,
                    stop_token_ids: Sequence[int] = ()) -> bool:
        if not isinstance(request, Request):
            request = Request(str(request), tuple(prompt_token_ids), max_new_tokens, temperature, seed,
                              tuple(stop_token_ids))
        return self.scheduler.add_request(request)

    def step(self) -> StepResult:
        return self.scheduler.step()

    def run_to_completion(self, max_steps: int = 100_000, overlap: bool = True) -> Dict[str, Tuple[int, ...]]:
        """Run until every request has finished.  With `overlap` (and no stop tokens, no recorded
        logits) the next step is decided and launched while the current one runs; decisions and
        tokens are those of stepping one by one."""
        if overlap and self.scheduler.can_overlap():
            self.scheduler.run_overlapped(max_steps)
            return {rid: tuple(seq.generated) for rid, seq in self.scheduler.finished.items()}
        return self.scheduler.run_to_completion(max_steps)

    def run_steps(self, count: int, overlap: bool = True) -> int:
        """At most `count` steps (fewer if nothing is left); returns how many ran."""
        if overlap and self.scheduler.can_overlap():
            return self.scheduler.run_overlapped(count, until_idle=False)
        done = 0
        while done < count and (self.scheduler.waiting or self.scheduler.running):
            self.scheduler.step()
            done += 1
        return done

    def events_of(self, kind: EventKind):
        return self.scheduler.events_of(kind)

    @property
    def finished(self):
        return self.scheduler.finished

    @property
    def rejected(self):
        return self.scheduler.rejected

    def generate(self, prompt_token_ids: Sequence[int], max_new_tokens: int, temperature: float = 0.0,
                 seed: int = 0, request_id: str = "generate") -> GenerationResult:
        """One request alone, to its end (greedy unless a temperature is given)."""
        if max_new_tokens < 1:
            raise ValueError(f"max_new_tokens must be at least 1, got {max_new_tokens}")
        if not prompt_token_ids:
            raise ValueError("prompt must be non-empty")
        if self.scheduler.waiting or self.scheduler.running:
            raise RuntimeError("generate() needs an idle engine")
        saved, self.record_logits = self.record_logits, True
        self.scheduler = self._new_scheduler()
        self.record_logits = saved
        if not self.add_request(Request(request_id, tuple(prompt_token_ids), max_new_tokens, temperature, seed)):
            raise ValueError(self.scheduler.events_of(EventKind.REJECT)[-1].detail)
        tokens = self.run_to_completion()[request_id]
        logits = torch.stack(self.scheduler.finished[request_id].step_logits)
        self.scheduler = self._new_scheduler()
        return GenerationResult(tuple(tokens), logits)

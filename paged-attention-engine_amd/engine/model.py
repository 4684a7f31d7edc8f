"""A model built from a plan: embedding, the scheduled blocks, final norm, head.

One body serves every way of calling it, as `_run_layers` does in the reference
(engine/model.py:322-351): embedding gather (:401,448), each scheduled block,
final norm (:351), selection of the wanted rows and the head product without
bias (:406,453-455).  The reference norms every row and then selects; the norm
is row-wise, so selecting first gives the same rows.  Logits are float32 in both
precisions.  `forward_pass_count` counts traversals of the schedule, the
reference's proof that a step is one pass (:180-186,338).
"""

from __future__ import annotations

from typing import Dict, List, Mapping, Optional, Tuple

import torch

from .. import models as _models  # noqa: F401  (registers the architectures)
from ..cache.manager import CacheManager, bytes_of_one_page_everywhere
from ..config.model_config import ModelPlan
from ..config.registry import read_config, read_config_dict
from ..kernels import lib as K
from ..parts import OwedRows, ResidualStream, StepContext, build_block, build_part
from ..parts.base import NORMS
from ..parts.linear import Linear
from ..weights.loader import load_weights
from ..weights.random_init import RandomWeights

TORCH_DTYPE = {"bfloat16": torch.bfloat16, "float32": torch.float32}
NAME_OF_DTYPE = {v: k for k, v in TORCH_DTYPE.items()}


def default_dtype(config) -> str:
    """The precision a model computes in when the caller names none: what its config.json says
    under `torch_dtype`, if that is one of the two the engine computes in; checkpoints stored in any
    other type (float16, say) are served in bfloat16."""
    stored = str(getattr(config, "torch_dtype", "") or "").replace("torch.", "")
    return stored if stored in TORCH_DTYPE else "bfloat16"


def plan_has_stops(plan: ModelPlan) -> bool:
    return len(plan.schedule) > 0


def _blocks_of(plan: ModelPlan, dtype, device):
    return [build_block(spec, dtype, device) for spec in plan.layers]


def expected_tensors(plan: ModelPlan) -> Dict[str, Tuple[int, ...]]:
    """Every checkpoint tensor the plan's parts declare, name -> shape."""
    out: Dict[str, Tuple[int, ...]] = {plan.embedding_name: (plan.vocab_size, plan.hidden_size)}
    for block in _blocks_of(plan, torch.float32, "meta"):
        out.update(block.tensors())
    out.update(build_part(NORMS, "norm", plan.final_norm, torch.float32, "meta").tensors(plan.final_norm_prefix))
    if plan.head_name is not None:
        out[plan.head_name] = (plan.vocab_size, plan.hidden_size)
    return out


class Model:
    def __init__(self, plan: ModelPlan, dtype: torch.dtype, device: str = "cuda:0") -> None:
        self.plan = plan
        self.dtype = dtype
        self.device = torch.device(device)
        self.blocks = _blocks_of(plan, dtype, self.device)
        self.final_norm = build_part(NORMS, "norm", plan.final_norm, dtype, self.device)
        self.embedding: Optional[torch.Tensor] = None
        self.head: Optional[Linear] = None
        self.forward_pass_count = 0

    # ------------------------------------------------------------------ weights
    def expected_tensors(self) -> Dict[str, Tuple[int, ...]]:
        return expected_tensors(self.plan)

    def optional_tensors(self) -> Tuple[str, ...]:
        return tuple(self.plan.optional_names)

    def bind(self, weights: Mapping[str, torch.Tensor]) -> None:
        plan = self.plan
        embedding = weights[plan.embedding_name]
        self.embedding = embedding.to(device=self.device, dtype=self.dtype).contiguous()
        for block in self.blocks:
            block.bind(weights)
        self.final_norm.bind(plan.final_norm_prefix, weights)
        if self.dtype == torch.bfloat16:
            K.skinny_tickets(self.device)  # made before any step is recorded as a graph
        if plan.head_name is None:
            self.head = Linear(self.embedding)  # tied: the same buffer, no second copy
        else:
            self.head = Linear(weights[plan.head_name].to(device=self.device, dtype=self.dtype).contiguous())

    @property
    def graph_max_rows(self) -> Optional[int]:
        """Most rows a step may hold and still be recorded as a HIP graph (None: any number), as the
        parts and the head's product say."""
        limits = [block.graph_max_rows for block in self.blocks if block.graph_max_rows is not None]
        if self.head is not None and self.head.graph_max_rows is not None:
            limits.append(self.head.graph_max_rows)
        return min(limits) if limits else None

    @property
    def graph_safe(self) -> bool:
        """Can a step of this model be recorded as a HIP graph?  Every part must launch device
        work from device-side data only, for some number of rows."""
        if not (all(block.graph_safe for block in self.blocks) and self.final_norm.graph_safe):
            return False
        return self.graph_max_rows is None or self.graph_max_rows > 0

    def step_list_parts(self, block_size: int) -> Dict[object, object]:
        """key -> the first part that asks for index lists under that key (see `Part.step_lists`)."""
        out: Dict[object, object] = {}
        for block in self.blocks:
            for part in getattr(block, "parts", lambda: [])():
                key = part.step_lists_key(block_size) if hasattr(part, "step_lists_key") else None
                if key is not None and key not in out:
                    out[key] = part
        return out

    # ------------------------------------------------------------------ cache needs
    def cache_specs(self):
        """(paged, states): per schedule stop, what it keeps per token / per request."""
        paged, states = [], []
        for entry in self.plan.schedule:
            mixer = self.blocks[entry.layer].mixer
            borrowed = entry.cache_from is not None
            paged.append(None if borrowed else mixer.paged_spec())
            states.append(None if borrowed else mixer.state_spec())
        return paged, states

    def page_bytes(self, block_size: int) -> int:
        """Bytes of one page in every cache group of this model (all stops)."""
        return bytes_of_one_page_everywhere(self.cache_specs()[0], block_size, self.dtype)

    def new_cache(self, block_size: int, num_blocks, num_slots: int) -> CacheManager:
        paged, states = self.cache_specs()
        return CacheManager(paged, states, block_size, num_blocks, num_slots, self.dtype, str(self.device))

    def decode_fusable(self, ctx: StepContext) -> bool:
        """Whether this step's blocks can run as one decode program: every sequence brings one token,
        and every scheduled block, and the final norm that takes over from the last, says it launches
        recordable kernels only at this many rows."""
        rows, bs = ctx.num_tokens, ctx.cache.block_size
        if rows != ctx.num_seqs or not plan_has_stops(self.plan):
            return False
        blocks = {entry.layer for entry in self.plan.schedule}
        return (all(getattr(self.blocks[i], "decode_fusable", lambda *_: False)(rows, bs) for i in blocks)
                and getattr(self.final_norm, "folded_for", lambda _: None)(rows) is not None)

    def max_program_phases(self) -> int:
        return 8 * len(self.plan.schedule) + 8

    def _run_blocks(self, ctx: StepContext, stream: ResidualStream, first_norms) -> None:
        for index, entry in enumerate(self.plan.schedule):
            ctx.entry = index
            ctx.cache_entry = index if entry.cache_from is None else entry.cache_from
            ctx.writes_cache = entry.cache_from is None
            stream.next_norm = first_norms[index + 1]
            self.blocks[entry.layer].forward(ctx, stream)

    # ------------------------------------------------------------------ forward
    def forward(self, ctx: StepContext, token_ids: torch.Tensor, logit_rows: torch.Tensor) -> torch.Tensor:
        """Run `token_ids` (int32 [T]) through the schedule once; float32 logits
        [len(logit_rows), vocab] at the flat rows `logit_rows` (int32)."""
        self.forward_pass_count += 1
        plan = self.plan
        T, H = ctx.num_tokens, plan.hidden_size
        residual = torch.empty((T, H), dtype=torch.float32, device=self.device)
        stream = ResidualStream(residual)
        # the norm that reads the stream first at every stop (and the final norm after the last)
        first_norms = [getattr(self.blocks[entry.layer], "mixer_norm", None) for entry in plan.schedule] + [self.final_norm]
        entry_fold = getattr(self.blocks[plan.schedule[0].layer], "entry_fold", None) if plan.schedule and T else None
        fold = entry_fold(T) if entry_fold is not None else None
        if fold is not None:
            # the first block's norm lets the embedding prepare its rows (see parts.OwedRows)
            norm, weight, eps = fold
            rows = torch.empty((T, H), dtype=torch.bfloat16, device=self.device)
            stats = torch.empty((T, K.stat_tiles(H)), dtype=torch.float32, device=self.device)
            K.embedding_rows(residual, self.embedding, token_ids, plan.embedding_scale, rows, weight, stats)
            stream.owed, stream.owed_to = OwedRows(rows, stats, eps), norm
        else:
            K.embedding(residual, self.embedding, token_ids, plan.embedding_scale)
        program = ctx.program if fold is not None and self.decode_fusable(ctx) else None
        if program is not None:
            # every block's kernels become phases of one resident kernel, which runs when all are recorded
            with K.recording(program):
                self._run_blocks(ctx, stream, first_norms)
            program.launch()
        else:
            self._run_blocks(ctx, stream, first_norms)
        rows = logit_rows.numel()
        if rows == 0:
            return torch.empty((0, plan.vocab_size), dtype=torch.float32, device=self.device)
        last = self.final_norm.forward(stream, logit_rows)
        logits = self.head.float32(last)
        if plan.logit_scale != 1.0 or plan.logit_softcap:
            K.logits_finish(logits, plan.logit_scale, plan.logit_softcap or 0.0)
        return logits


def load_model(model_dir: str, dtype: Optional[str] = None, device: str = "cuda:0") -> Model:
    """The model of a folder with config.json and safetensors weights; the class
    of model is chosen by config.json's `architectures`, and so is the precision if `dtype` is None
    (`default_dtype`)."""
    config = read_config(model_dir)
    if dtype is None:
        dtype = default_dtype(config)
    if dtype not in TORCH_DTYPE:
        raise ValueError(f"dtype must be 'bfloat16' or 'float32', got {dtype!r}")
    model = Model(config.plan(), TORCH_DTYPE[dtype], device)
    model.config = config
    weights = load_weights(model_dir, model.expected_tensors(), model.optional_tensors())
    model.bind(weights)
    return model


def random_model(config, seed: int = 0, dtype: Optional[str] = None, device: str = "cuda:0", std: float = 0.02,
                 norm_std: float = 0.0) -> Model:
    """A model of `config` (a config.json dict, or a registered architecture's typed config) with
    random weights drawn on the device, tensor by tensor as the parts bind them: nothing is written
    to disk and no tensor exists twice, so the 72B shape's 145 GB fit one GPU.  The reference draws
    random weights only for its tiny test model (tests/tiny_model.py:21-50)."""
    if isinstance(config, Mapping):
        config = read_config_dict(config)
    if dtype is None:
        dtype = default_dtype(config)
    if dtype not in TORCH_DTYPE:
        raise ValueError(f"dtype must be 'bfloat16' or 'float32', got {dtype!r}")
    model = Model(config.plan(), TORCH_DTYPE[dtype], device)
    model.config = config
    model.bind(RandomWeights(model.expected_tensors(), seed, std, norm_std, device))
    return model

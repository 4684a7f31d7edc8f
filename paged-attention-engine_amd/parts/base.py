"""What a part is, what it sees of a step, and the registries parts are found in.

A model is put together from five kinds of parts, each chosen by the `kind` of
its spec and none aware of the model it sits in:

  norm               forward(stream, rows=None) -> normalised activations
  position encoding  encode(ctx, x, num_heads, head_dim): encodes heads in place by the tokens' positions
  mixer              forward(ctx, x) -> y        (attention here; keeps what it caches, paged or per request)
  feed-forward       forward(ctx, x) -> y
  block              forward(ctx, stream)        (arranges two norms, a mixer and a feed-forward)

Each part declares the tensors it needs (`tensors(prefix)`: name -> shape) and
takes them in `bind(prefix, weights)`.  The reference wires the same pieces by
hand inside one class (engine/model.py:281-351) and lets its attention backends
vary behind `attend(layer, q, k, v)` (engine/attention.py:248-277); the registry
and the spec-driven construction are this engine's own.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, Dict, List, Mapping, Optional, Tuple

import torch


class ScaleShape(tuple):
    """The declared shape of a tensor that multiplies activations elementwise (a norm's weight).
    Equal to the plain tuple; random mode reads `centre` and draws such a tensor about one instead
    of about zero.  A part marks the tensor where it declares it, whatever the tensor is called."""

    centre = 1.0


class OwedRows:
    """Activations whose division by their root mean square is still owed.

    `rows` = bfloat16(x * w) for the input x and the weight w of a norm; `stats[m]` holds shares
    that add up to sum(x[m]^2) (one per 16 columns).  norm(x) W^T = rsqrt(mean(x^2) + eps) *
    (rows W^T), so a matrix product can pay the scale on its finished sums, and a decode step
    needs no norm kernel between its products.  A part that wants plain activations calls
    `settle()`."""

    def __init__(self, rows: torch.Tensor, stats: torch.Tensor, eps: float) -> None:
        self.rows, self.stats, self.eps = rows, stats, eps

    @property
    def shape(self):
        return self.rows.shape

    @property
    def dtype(self):
        return self.rows.dtype

    @property
    def device(self):
        return self.rows.device

    @property
    def row_scale(self):
        return self.stats, self.eps

    def settle(self) -> torch.Tensor:
        from ..kernels import lib as K
        return K.scaled_rows(self.rows, self.stats, self.eps)


def plain_rows(x):
    """`x` as plain activations, whatever form it came in."""
    return x.settle() if isinstance(x, OwedRows) else x


class ResidualStream:
    """The float32 residual sum of a step and the branch output not yet added to it.

    Norm parts add `pending` while they normalise, so the sum is formed in
    32-bit and written once.  A branch whose last product can add itself into the residual
    (see `BranchSink`) leaves no `pending` but `owed`, the rows prepared for the norm `owed_to`."""

    def __init__(self, residual: torch.Tensor) -> None:
        self.residual = residual
        self.pending: Optional[torch.Tensor] = None
        self.owed: Optional[OwedRows] = None
        self.owed_to: Optional[object] = None
        self.next_norm: Optional[object] = None  # set by the model: the norm that reads the stream after this block


class BranchSink:
    """Where a branch's last product may deliver itself instead of returning its output: added
    into the stream's residual in place, with the rows the following norm's consumer wants
    prepared on the way.  `norm` is the norm part that will read the stream next; it must offer
    `folded_for(rows) -> (weight, eps) | None` for the offer to be taken up."""

    def __init__(self, stream: ResidualStream, norm) -> None:
        self.stream, self.norm = stream, norm

    def folded(self, rows: int):
        fold = getattr(self.norm, "folded_for", None)
        return fold(rows) if fold is not None else None

    def deliver(self, owed: OwedRows) -> None:
        self.stream.pending = None
        self.stream.owed, self.stream.owed_to = owed, self.norm


@dataclass(frozen=True)
class StepShape:
    """A step on the host, before anything is on the device: which sequences bring how many
    tokens at which place.  Parts that want index lists of their own for a step (work lists of
    a kernel, say) build them from this; see `Part.step_lists`."""

    seq_ids: Tuple[int, ...]
    q_starts: Tuple[int, ...]   # first flat row of each sequence
    q_lens: Tuple[int, ...]     # rows of each sequence in this step
    past_lens: Tuple[int, ...]  # tokens each sequence held before the step
    block_size: int

    @property
    def num_tokens(self) -> int:
        return sum(self.q_lens)


@dataclass
class StepContext:
    """One step as parts see it: flat tokens of several sequences and their caches."""

    dtype: torch.dtype                 # storage type of activations that feed matrix products
    device: torch.device
    num_tokens: int
    num_seqs: int
    positions: torch.Tensor            # int32 [T] position of each token in its sequence
    tok_seq: torch.Tensor              # int32 [T] row of each token's sequence in the tables below
    block_tables: Dict[int, torch.Tensor]  # cache group -> int32 [S, max_blocks]
    slots: torch.Tensor                # int32 [S] state slot of each sequence
    cache: "object"                    # the CacheManager
    # the same on the host, for parts that loop over sequences
    seq_ids: List[int] = field(default_factory=list)
    q_starts: List[int] = field(default_factory=list)   # first flat row of each sequence
    q_lens: List[int] = field(default_factory=list)     # rows of each sequence in this step
    past_lens: List[int] = field(default_factory=list)  # tokens each sequence held before the step
    host_slots: List[int] = field(default_factory=list)
    # set by the model for the stop that is running
    entry: int = 0                     # index in the schedule
    cache_entry: int = 0               # the stop whose cache is read (entry itself unless it borrows)
    writes_cache: bool = True
    sink: Optional["BranchSink"] = None  # set by the block around a branch: see BranchSink
    # room for the step's layers as one resident kernel (kernels.lib.DecodeProgram), offered by the step
    # function for steps in which every sequence brings one token; None: every kernel is launched by itself
    program: Optional[object] = None
    # what a part computes once per step for every layer that has the same part (a table of angles,
    # say), under a key of the part's choosing; the step function also leaves here, under
    # `step_lists_key`, the index lists a part asked for (`Part.step_lists`), as int32 device tensors
    memo: Dict[object, object] = field(default_factory=dict)


class Part:
    """Base of all parts: holds its spec and the precision it computes in."""

    # True when `forward` only launches work on the current stream with device-side
    # data (nothing read from the context's host lists, no synchronisation): such a
    # part can be recorded into a HIP graph and replayed with new inputs.
    graph_safe = False
    # The most rows of a step for which that holds (None: any number): a part whose products
    # leave this engine's kernels above some row count says so here.
    graph_max_rows: Optional[int] = None
    # True when `forward` takes its input as `OwedRows` as well as a plain tensor (the block
    # settles them for parts that do not).
    takes_owed_rows = False

    def decode_fusable(self, rows: int, block_size: int) -> bool:
        """Whether, in a step of `rows` sequences that bring one token each, `forward` does all of its
        device work through wrappers that a decode program can record (see kernels.lib.recording):
        the few-row products and the decode attention.  A part that launches anything else, or calls
        the platform's libraries, must say no (the default)."""
        return False

    def __init__(self, spec, dtype: torch.dtype, device) -> None:
        self.spec = spec
        self.dtype = dtype
        self.device = device

    def tensors(self, prefix: str) -> Dict[str, Tuple[int, ...]]:
        """Checkpoint tensors this part needs, by full name."""
        return {}

    def bind(self, prefix: str, weights: Mapping[str, torch.Tensor]) -> None:
        """Take the tensors declared by `tensors(prefix)` out of `weights`."""

    def matrix(self, t: torch.Tensor) -> torch.Tensor:
        """A matrix-product operand in the compute precision, on the device."""
        return t.to(device=self.device, dtype=self.dtype).contiguous()

    def vector(self, t: torch.Tensor) -> torch.Tensor:
        """A norm weight or bias: stays float32 if stored so, else the compute precision."""
        keep = torch.float32 if t.dtype == torch.float32 else self.dtype
        return t.to(device=self.device, dtype=keep).contiguous()

    # Index lists of the part's own for every step (a kernel's work lists, for instance).  A part
    # that wants them names a key (parts with equal keys share one set of lists per step) and
    # builds them on the host from the step's shape: {name: (flat list of ints, row width or 0)}.
    # The step function copies them to the device with its own metadata, in the same transfer,
    # and leaves {name: int32 tensor} in `ctx.memo[key]` (viewed [-1, width] when a width is given).
    def step_lists_key(self, block_size: int):
        return None

    def step_lists(self, shape: "StepShape"):
        return {}

    # what the part keeps in the cache (mixers override)
    def paged_spec(self):
        return None

    def state_spec(self):
        return None


# kind -> class, one registry per role
NORMS: Dict[str, Callable] = {}
POSITION_ENCODINGS: Dict[str, Callable] = {}
MIXERS: Dict[str, Callable] = {}
FEED_FORWARDS: Dict[str, Callable] = {}
BLOCKS: Dict[str, Callable] = {}


def _register(table: Dict[str, Callable], kind: str):
    def wrap(cls):
        table[kind] = cls
        return cls
    return wrap


def register_norm(kind: str):
    return _register(NORMS, kind)


def register_position_encoding(kind: str):
    return _register(POSITION_ENCODINGS, kind)


def register_mixer(kind: str):
    return _register(MIXERS, kind)


def register_feed_forward(kind: str):
    return _register(FEED_FORWARDS, kind)


def register_block(kind: str):
    return _register(BLOCKS, kind)


def build_part(table: Dict[str, Callable], role: str, spec, dtype, device):
    if spec.kind not in table:
        raise KeyError(f"no {role} of kind '{spec.kind}' is registered; known: {', '.join(sorted(table))}")
    return table[spec.kind](spec, dtype, device)

"""Typed descriptions of a model: specs of parts, layers, and the order they run in.

Nothing here knows an architecture.  An architecture's own config class (for
Qwen2: `models/qwen2.py`) reads its config.json keys and turns them into a
`ModelPlan`; the engine builds parts from the plan's specs by their `kind`.

The reference keeps the same constants in one frozen dataclass, `ModelDims`
(engine/model.py:43-80), and passes eps, theta, scale and group size to free
functions as arguments (engine/model.py:117,132,138; engine/attention.py:135-144).
Here every part's spec carries its own sizes and constants so that two layers of
one model may differ.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Mapping, Optional, Tuple


class ConfigError(ValueError):
    """A config.json that cannot be turned into a model, with the key named."""


@dataclass(frozen=True)
class PartSpec:
    """Base of every spec: `kind` selects the implementation in the part registry."""

    kind: str


@dataclass(frozen=True)
class NormSpec(PartSpec):
    size: int = 0
    eps: float = 0.0
    kind: str = "rmsnorm"
    weight_name: str = "weight"  # the tensor's name below the norm's prefix


@dataclass(frozen=True)
class PositionSpec(PartSpec):
    """Rotation of query and key by absolute position; `rotary_dim` leading
    features of each head are rotated in pairs (i, i + rotary_dim/2)."""

    rotary_dim: int = 0
    theta: float = 10000.0
    kind: str = "neox_rope"


@dataclass(frozen=True)
class MixerSpec(PartSpec):
    """Causal attention over the paged cache with grouped key/value heads.

    `window` None means every earlier key; otherwise a query at position p sees
    keys p-window+1 .. p.  `scale` multiplies the scores."""

    hidden_size: int = 0
    num_heads: int = 0
    num_kv_heads: int = 0
    head_dim: int = 0
    scale: float = 1.0
    qkv_bias: bool = True
    out_bias: bool = False
    window: Optional[int] = None
    position: Optional[PositionSpec] = None
    kind: str = "attention"
    # names of the four projections below the mixer's prefix (each with ".weight" and, where the
    # spec says so, ".bias"): an architecture that calls them otherwise sets these, not a new mixer
    q_name: str = "q_proj"
    k_name: str = "k_proj"
    v_name: str = "v_proj"
    o_name: str = "o_proj"


@dataclass(frozen=True)
class FeedForwardSpec(PartSpec):
    hidden_size: int = 0
    intermediate_size: int = 0
    activation: str = "silu"
    kind: str = "swiglu"
    # names of the three projections below the feed-forward's prefix
    gate_name: str = "gate_proj"
    up_name: str = "up_proj"
    down_name: str = "down_proj"


@dataclass(frozen=True)
class LayerSpec:
    """One block: which parts, in which arrangement, under which tensor-name prefix."""

    prefix: str
    mixer: PartSpec
    feed_forward: PartSpec
    mixer_norm: PartSpec
    feed_forward_norm: PartSpec
    # tensor-name prefixes of the four parts below `prefix`
    mixer_prefix: str = "self_attn."
    feed_forward_prefix: str = "mlp."
    mixer_norm_prefix: str = "input_layernorm."
    feed_forward_norm_prefix: str = "post_attention_layernorm."
    arrangement: str = "prenorm"


@dataclass(frozen=True)
class ScheduleEntry:
    """One stop of the forward pass.

    `layer` indexes `ModelPlan.layers` (a layer may be named by several
    entries: its weights are then shared while each entry keeps a cache of its
    own).  `cache_from` names an earlier *entry* whose cache this entry reads
    instead of writing one."""

    layer: int
    cache_from: Optional[int] = None


@dataclass(frozen=True)
class ModelPlan:
    architecture: str
    hidden_size: int
    vocab_size: int
    layers: Tuple[LayerSpec, ...]
    schedule: Tuple[ScheduleEntry, ...]
    final_norm: PartSpec
    embedding_name: str
    head_name: Optional[str]  # None: the head shares the embedding matrix
    final_norm_prefix: str
    max_positions: Optional[int] = None
    # tensors a checkpoint of this architecture may hold without the model using them (a head stored
    # although it is tied to the embedding, say): the loader passes over them
    optional_names: Tuple[str, ...] = ()
    # what some architectures do around the blocks (the reference's model does none of it:
    # engine/model.py:401,453-455 gathers rows and multiplies by the head as they are)
    embedding_scale: float = 1.0            # the gathered rows are multiplied by this
    logit_scale: float = 1.0                # the logits are multiplied by this ...
    logit_softcap: Optional[float] = None   # ... and then, with a cap c, become c * tanh(logits / c)
    extra: Mapping[str, Any] = field(default_factory=dict)

    def __post_init__(self) -> None:
        for i, entry in enumerate(self.schedule):
            if not 0 <= entry.layer < len(self.layers):
                raise ConfigError(f"schedule entry {i} names layer {entry.layer} of {len(self.layers)}")
            if entry.cache_from is not None and not 0 <= entry.cache_from < i:
                raise ConfigError(
                    f"schedule entry {i} reads the cache of entry {entry.cache_from}, "
                    "which is not an earlier entry")
        if self.logit_softcap is not None and not self.logit_softcap > 0:
            raise ConfigError(f"logit_softcap must be positive, got {self.logit_softcap}")


def require(cfg: Mapping[str, Any], key: str, kind=int):
    """Fetch a required config.json key with a typed, named error."""
    if key not in cfg or cfg[key] is None:
        raise ConfigError(f"config.json lacks the key '{key}'")
    try:
        return kind(cfg[key])
    except (TypeError, ValueError) as err:
        raise ConfigError(f"config.json key '{key}' = {cfg[key]!r} is not {kind.__name__}") from err


def positive(name: str, value) -> None:
    if value <= 0:
        raise ConfigError(f"config.json key '{name}' must be positive, got {value}")

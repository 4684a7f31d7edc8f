"""Qwen2 / Qwen2.5 dense decoder: its config.json keys and the plan they give.

The reference reads the same constants from a live transformers config object
(`ModelDims.from_config`, engine/model.py:64-80): num_hidden_layers,
num_attention_heads, num_key_value_heads, head_dim (falling back to
hidden_size // num_attention_heads), hidden_size, rms_norm_eps, vocab_size and
rope_theta (as rope_parameters["rope_theta"]).  It takes the intermediate size
and the tying of the head from the weights (engine/model.py:220-222); here both
are config keys, checked against the file by the loader.

Fixed by the architecture, as in the reference: bias on q/k/v and none on o
(engine/model.py:87-92,303-305,315); rotation of pairs (i, i + hd/2) over the
whole head (:126-129,148-161); scores scaled by head_dim ** -0.5 (:60-62);
SiLU-gated feed-forward without bias (:317-320); pre-norm residual blocks and
a final norm (:340-351); tensor names of the checkpoint (:198-227).

The reference attends over every earlier key in every layer
(engine/attention.py:474-487).  A config with `use_sliding_window` true gives the
layers from `max_window_layers` on a window of `sliding_window` keys; that reading
of the keys is this engine's own.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional

from ..config.model_config import (ConfigError, FeedForwardSpec, LayerSpec, MixerSpec, ModelPlan,
                                   NormSpec, PositionSpec, ScheduleEntry, positive, require)
from ..config.registry import register_architecture

ARCHITECTURE = "Qwen2ForCausalLM"


@dataclass(frozen=True)
class Qwen2Config:
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    rms_norm_eps: float
    rope_theta: float
    tie_word_embeddings: bool
    max_position_embeddings: Optional[int]
    use_sliding_window: bool
    sliding_window: Optional[int]
    max_window_layers: int
    hidden_act: str = "silu"
    torch_dtype: str = "bfloat16"

    @classmethod
    def from_dict(cls, cfg: Mapping[str, Any]) -> "Qwen2Config":
        hidden = require(cfg, "hidden_size")
        heads = require(cfg, "num_attention_heads")
        positive("hidden_size", hidden)
        positive("num_attention_heads", heads)
        head_dim = cfg.get("head_dim") or hidden // heads
        if "rope_theta" in cfg and cfg["rope_theta"] is not None:
            theta = float(cfg["rope_theta"])
        elif isinstance(cfg.get("rope_parameters"), Mapping) and "rope_theta" in cfg["rope_parameters"]:
            theta = float(cfg["rope_parameters"]["rope_theta"])
        else:
            raise ConfigError("config.json lacks the key 'rope_theta'")
        scaling = cfg.get("rope_scaling")
        if scaling not in (None, {}) and scaling.get("rope_type", scaling.get("type")) not in (None, "default"):
            raise ConfigError(f"rope_scaling {scaling!r} is not supported (only the default rope type)")
        act = cfg.get("hidden_act", "silu")
        if act != "silu":
            raise ConfigError(f"hidden_act '{act}' is not supported (only 'silu')")
        layers = require(cfg, "num_hidden_layers")
        use_window = bool(cfg.get("use_sliding_window", False))
        window = cfg.get("sliding_window")
        if use_window and not window:
            raise ConfigError("use_sliding_window is true but config.json lacks 'sliding_window'")
        out = cls(
            vocab_size=require(cfg, "vocab_size"),
            hidden_size=hidden,
            intermediate_size=require(cfg, "intermediate_size"),
            num_hidden_layers=layers,
            num_attention_heads=heads,
            num_key_value_heads=int(cfg.get("num_key_value_heads") or heads),
            head_dim=int(head_dim),
            rms_norm_eps=require(cfg, "rms_norm_eps", float),
            rope_theta=theta,
            tie_word_embeddings=bool(cfg.get("tie_word_embeddings", False)),
            max_position_embeddings=(int(cfg["max_position_embeddings"])
                                     if cfg.get("max_position_embeddings") else None),
            use_sliding_window=use_window,
            sliding_window=int(window) if window else None,
            max_window_layers=int(cfg.get("max_window_layers", layers)),
            hidden_act=act,
            torch_dtype=str(cfg.get("torch_dtype", cfg.get("dtype", "bfloat16"))),
        )
        out.validate()
        return out

    def validate(self) -> None:
        for name in ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                     "num_attention_heads", "num_key_value_heads", "head_dim"):
            positive(name, getattr(self, name))
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"num_attention_heads {self.num_attention_heads} is not a multiple of "
                f"num_key_value_heads {self.num_key_value_heads}")
        if self.head_dim % 2:
            raise ConfigError(f"head_dim {self.head_dim} must be even for rotary pairs")
        if not self.rms_norm_eps > 0:
            raise ConfigError(f"rms_norm_eps must be positive, got {self.rms_norm_eps}")
        if not self.rope_theta > 0:
            raise ConfigError(f"rope_theta must be positive, got {self.rope_theta}")
        if self.use_sliding_window and self.sliding_window < 1:
            raise ConfigError(f"sliding_window must be positive, got {self.sliding_window}")

    def window_of(self, layer: int) -> Optional[int]:
        if self.use_sliding_window and layer >= self.max_window_layers:
            return self.sliding_window
        return None

    def to_json_dict(self) -> dict:
        return {
            "architectures": [ARCHITECTURE],
            "model_type": "qwen2",
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "hidden_act": self.hidden_act,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "tie_word_embeddings": self.tie_word_embeddings,
            "max_position_embeddings": self.max_position_embeddings,
            "use_sliding_window": self.use_sliding_window,
            "sliding_window": self.sliding_window,
            "max_window_layers": self.max_window_layers,
            "torch_dtype": self.torch_dtype,
        }

    def plan(self) -> ModelPlan:
        norm = NormSpec(size=self.hidden_size, eps=self.rms_norm_eps)
        rope = PositionSpec(rotary_dim=self.head_dim, theta=self.rope_theta)
        ffn = FeedForwardSpec(hidden_size=self.hidden_size,
                              intermediate_size=self.intermediate_size, activation=self.hidden_act)
        layers = []
        for i in range(self.num_hidden_layers):
            mixer = MixerSpec(
                hidden_size=self.hidden_size, num_heads=self.num_attention_heads,
                num_kv_heads=self.num_key_value_heads, head_dim=self.head_dim,
                scale=self.head_dim ** -0.5, qkv_bias=True, out_bias=False,
                window=self.window_of(i), position=rope)
            layers.append(LayerSpec(prefix=f"model.layers.{i}.", mixer=mixer, feed_forward=ffn,
                                    mixer_norm=norm, feed_forward_norm=norm))
        return ModelPlan(
            architecture=ARCHITECTURE,
            hidden_size=self.hidden_size,
            vocab_size=self.vocab_size,
            layers=tuple(layers),
            schedule=tuple(ScheduleEntry(layer=i) for i in range(self.num_hidden_layers)),
            final_norm=norm,
            embedding_name="model.embed_tokens.weight",
            head_name=None if self.tie_word_embeddings else "lm_head.weight",
            final_norm_prefix="model.norm.",
            max_positions=self.max_position_embeddings,
            # a file of a model with a tied head may still store the head
            optional_names=("lm_head.weight",) if self.tie_word_embeddings else (),
        )


register_architecture(ARCHITECTURE, Qwen2Config.from_dict)

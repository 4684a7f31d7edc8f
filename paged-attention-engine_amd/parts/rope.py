"""Rotary position encoding (pairs (i, i + rot/2)).

inv_freq[i] = 1 / theta ** (2 i / rot), built exactly as the reference builds it
(engine/model.py:132-135: int64 arange -> float, divided by the size, theta to
that power, in float32); angle = position * inv_freq in float32
(engine/model.py:138-152); out = x * cos + rotate_half(x) * sin (:126-129,155-161).
The reference casts cos and sin to the activation type before the multiply; here
they stay float32 and the result is rounded once.

A position encoding encodes heads in place (`encode`) and knows nothing of caches:
storing keys and values is the mixer's business.  An encoding that is a rotation by a
table of cosines and sines may also hand out that table (`rotary_table`), which lets a
mixer run the rotation inside its own fused kernels.
"""

from __future__ import annotations

import torch

from ..kernels import lib as K
from .base import Part, register_position_encoding


@register_position_encoding("neox_rope")
class NeoxRope(Part):
    graph_safe = True

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        rot = spec.rotary_dim
        if rot % 2:
            raise ValueError(f"rotary_dim {rot} must be even")
        exponent = torch.arange(0, rot, 2, dtype=torch.int64).to(torch.float32)
        self.inv_freq = (1.0 / (spec.theta ** (exponent / rot))).to(device)

    def rotary_table(self, ctx):
        """(rotated width, cosines and sines [T, width / 2, 2] of every token's angles): computed by
        the first layer of a step that asks and shared by all layers with the same rotation."""
        rot = self.spec.rotary_dim
        if not rot:
            return 0, None
        key = ("neox_rope", rot, self.spec.theta)
        table = ctx.memo.get(key)
        if table is None:
            table = ctx.memo[key] = K.rope_table(ctx.positions, self.inv_freq)
        return rot, table

    def encode(self, ctx, x: torch.Tensor, num_heads: int, head_dim: int) -> None:
        """Rotate the first `num_heads` heads of every row of `x` in place."""
        rot, table = self.rotary_table(ctx)
        if rot:
            K.rotate_heads(x, num_heads, head_dim, rot, table, ctx.positions)


@register_position_encoding("none")
class NoPosition(Part):
    """No encoding: queries and keys stay as they are."""

    graph_safe = True

    def rotary_table(self, ctx):
        return 0, None

    def encode(self, ctx, x: torch.Tensor, num_heads: int, head_dim: int) -> None:
        return None

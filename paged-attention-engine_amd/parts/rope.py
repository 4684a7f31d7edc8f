"""Rotary position encoding (pairs (i, i + rot/2)), fused with the cache write.

inv_freq[i] = 1 / theta ** (2 i / rot), built exactly as the reference builds it
(engine/model.py:132-135: int64 arange -> float, divided by the size, theta to
that power, in float32); angle = position * inv_freq in float32
(engine/model.py:138-152); out = x * cos + rotate_half(x) * sin (:126-129,155-161).
The reference casts cos and sin to the activation type before the multiply; here
they stay float32 and the result is rounded once.
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

    def cos_sin(self, ctx):
        """Cosines and sines of every token's angles, computed by the first layer of a step that
        asks and shared by all layers with the same rotation."""
        if not self.spec.rotary_dim:
            return None
        key = ("neox_rope", self.spec.rotary_dim, self.spec.theta)
        table = ctx.memo.get(key)
        if table is None:
            table = ctx.memo[key] = K.rope_table(ctx.positions, self.inv_freq)
        return table

    def encode_and_store(self, ctx, qkv, nh, nkv, hd, k_cache, v_cache, block_table, block_size):
        """Rotate the query heads of `qkv` in place; write rotated keys and raw
        values to the cache (when `k_cache` is given)."""
        K.rope_kv_write(qkv, nh, nkv, hd, self.spec.rotary_dim, self.cos_sin(ctx), ctx.positions, ctx.tok_seq,
                        block_table, block_size, k_cache, v_cache)

    def project_encode_store(self, ctx, x, linear, nh, nkv, hd, k_cache, v_cache, block_table, block_size):
        """The projection, the rotation and the cache write as one kernel, where there is one for
        these sizes; otherwise None, and the caller runs the two steps."""
        if x.dtype != torch.bfloat16 or not K.skinny_rope_supported(x, linear.weight, hd, self.spec.rotary_dim):
            return None
        return _fused_projection(self.spec.rotary_dim, self.cos_sin(ctx), ctx, x, linear, nh, nkv, hd, k_cache,
                                 v_cache, block_table, block_size)


def _fused_projection(rot, cos_sin, ctx, x, linear, nh, nkv, hd, k_cache, v_cache, block_table, block_size):
    q = torch.empty((x.shape[0], nh * hd), dtype=x.dtype, device=x.device)
    splits = K.whole_sum_splits(linear.out_features, linear.in_features, x.shape[0])
    K.gemm_skinny_rope(q, x, linear.weight, linear.bias, nh, nkv, hd, rot, cos_sin, ctx.positions, ctx.tok_seq,
                       block_table, block_size, k_cache, v_cache, splits)
    return q


@register_position_encoding("none")
class NoPosition(Part):
    graph_safe = True
    """No encoding: keys and values go to the cache as they are."""

    def encode_and_store(self, ctx, qkv, nh, nkv, hd, k_cache, v_cache, block_table, block_size):
        if k_cache is not None:
            K.rope_kv_write(qkv, nh, nkv, hd, 0, None, ctx.positions, ctx.tok_seq, block_table, block_size,
                            k_cache, v_cache)

    def project_encode_store(self, ctx, x, linear, nh, nkv, hd, k_cache, v_cache, block_table, block_size):
        if x.dtype != torch.bfloat16 or not K.skinny_rope_supported(x, linear.weight, hd, 0):
            return None
        return _fused_projection(0, None, ctx, x, linear, nh, nkv, hd, k_cache, v_cache, block_table, block_size)

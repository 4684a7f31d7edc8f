"""Causal attention with grouped key/value heads over the paged cache.

Per layer, as in the reference (engine/model.py:281-315): q/k/v projections
(with bias if the spec says so), split into heads of `head_dim` (head j = output
features [j*hd, (j+1)*hd)), position encoding of q and k, new keys and values
stored at their cache slots, attention of every query over the sequence's keys
up to its own position (engine/attention.py:474-487), heads merged, output
projection.  The three projections are one product over concatenated weights;
row-wise dot products are unchanged by the concatenation.

A stop that borrows another stop's cache projects queries only and reads keys
and values written by the owner.
"""

from __future__ import annotations

import torch

from ..cache.manager import PagedSpec
from ..kernels import lib as K
from .base import POSITION_ENCODINGS, Part, build_part, register_mixer
from .linear import Linear


@register_mixer("attention")
class PagedAttention(Part):
    @property
    def graph_safe(self) -> bool:
        return self.position.graph_safe
    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        if spec.num_heads % spec.num_kv_heads:
            raise ValueError(f"{spec.num_heads} query heads over {spec.num_kv_heads} key/value heads")
        if spec.head_dim % 16 or not 16 <= spec.head_dim <= 256:
            raise ValueError(f"head_dim {spec.head_dim}: the attention kernels take multiples of 16 up to 256")
        self.position = (build_part(POSITION_ENCODINGS, "position encoding", spec.position, dtype, device)
                         if spec.position is not None else
                         POSITION_ENCODINGS["none"](None, dtype, device))

    def product_widths(self):
        return [self.spec.hidden_size, self.spec.num_heads * self.spec.head_dim]

    def paged_spec(self):
        return PagedSpec(self.spec.num_kv_heads, self.spec.head_dim, self.spec.window)

    def tensors(self, prefix):
        s = self.spec
        out = {prefix + "q_proj.weight": (s.num_heads * s.head_dim, s.hidden_size),
               prefix + "k_proj.weight": (s.num_kv_heads * s.head_dim, s.hidden_size),
               prefix + "v_proj.weight": (s.num_kv_heads * s.head_dim, s.hidden_size),
               prefix + "o_proj.weight": (s.hidden_size, s.num_heads * s.head_dim)}
        if s.qkv_bias:
            out[prefix + "q_proj.bias"] = (s.num_heads * s.head_dim,)
            out[prefix + "k_proj.bias"] = (s.num_kv_heads * s.head_dim,)
            out[prefix + "v_proj.bias"] = (s.num_kv_heads * s.head_dim,)
        if s.out_bias:
            out[prefix + "o_proj.bias"] = (s.hidden_size,)
        return out

    def bind(self, prefix, weights):
        s = self.spec
        names = ("q_proj", "k_proj", "v_proj")
        w = torch.cat([weights[prefix + n + ".weight"] for n in names], dim=0)
        b = (torch.cat([weights[prefix + n + ".bias"] for n in names], dim=0) if s.qkv_bias else None)
        self.qkv = Linear(self.matrix(w), None if b is None else self.vector(b))
        nq = s.num_heads * s.head_dim
        self.q_only = Linear(self.qkv.weight[:nq], None if b is None else self.qkv.bias[:nq])
        ob = weights.get(prefix + "o_proj.bias") if s.out_bias else None
        self.out = Linear(self.matrix(weights[prefix + "o_proj.weight"]), None if ob is None else self.vector(ob))

    def forward(self, ctx, x: torch.Tensor) -> torch.Tensor:
        s = self.spec
        group = ctx.cache.group_of(ctx.cache_entry)
        k_cache, v_cache = ctx.cache.kv_of(ctx.cache_entry)
        table = ctx.block_tables[group]
        # a position encoding may offer the projection, its encoding and the cache write as one step
        fused = getattr(self.position, "project_encode_store", None)
        if ctx.writes_cache:
            stored = (s.num_kv_heads, s.head_dim, k_cache, v_cache, table, ctx.cache.block_size)
            qkv = fused(ctx, x, self.qkv, s.num_heads, *stored) if fused else None
            if qkv is None:
                qkv = self.qkv(x)
                self.position.encode_and_store(ctx, qkv, s.num_heads, *stored)
        else:
            stored = (0, s.head_dim, None, None, None, ctx.cache.block_size)
            qkv = fused(ctx, x, self.q_only, s.num_heads, *stored) if fused else None
            if qkv is None:
                qkv = self.q_only(x)
                self.position.encode_and_store(ctx, qkv, s.num_heads, *stored)
        attn = torch.empty((x.shape[0], s.num_heads * s.head_dim), dtype=x.dtype, device=x.device)
        geometry = (s.num_heads, s.num_kv_heads, s.head_dim, s.scale, s.window or 0)
        if K.mfma_attention_supported(x.dtype, s.num_heads, s.num_kv_heads, s.head_dim, ctx.cache.block_size) \
                and ctx.decode_tokens is not None:
            if ctx.decode_tokens.numel():
                K.attn_decode(attn, qkv, k_cache, v_cache, ctx.decode_tokens, ctx.positions, ctx.tok_seq, table,
                              *geometry)
            if ctx.prefill_tiles.numel():
                K.attn_prefill(attn, qkv, k_cache, v_cache, ctx.prefill_tiles, ctx.positions, table, *geometry)
        else:
            K.paged_attention_generic(attn, qkv, k_cache, v_cache, ctx.positions, ctx.tok_seq, table, *geometry)
        return self.out.branch(attn)

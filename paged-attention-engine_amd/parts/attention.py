"""Causal attention with grouped key/value heads over the paged cache.

Per layer, as in the reference (engine/model.py:281-315): q/k/v projections
(with bias if the spec says so), split into heads of `head_dim` (head j = output
features [j*hd, (j+1)*hd)), position encoding of q and k, new keys and values
stored at their cache slots, attention of every query over the sequence's keys
up to its own position (engine/attention.py:474-487), heads merged, output
projection.  The three projections are one product over concatenated weights;
row-wise dot products are unchanged by the concatenation.

The mixer owns its cache: it declares the pages it keeps (`paged_spec`), stores new
keys and values itself, and builds the work lists of its kernels from the step's shape
(`step_lists`).  The position encoding only encodes; when it is a rotation that hands
out its table, the rotation runs inside the mixer's fused kernels (projection +
rotation + store for up to 64 rows, rotation + store above).

A stop that borrows another stop's cache projects queries only and reads keys
and values written by the owner.
"""

from __future__ import annotations

import torch

from ..cache.manager import attention_pages
from ..kernels import lib as K
from .base import POSITION_ENCODINGS, OwedRows, Part, StepShape, build_part, plain_rows, register_mixer
from .linear import Linear, rows_a_graph_may_hold

WORK_LISTS = ("paged attention work lists", K.PREFILL_TILE)


def attention_work_lists(shape: StepShape):
    """What the matrix-core attention kernels walk: `decode_work`, one (flat row, position, table
    row, 0) for every sequence that brings one token (all a workgroup needs to know of its token in
    one 16-byte load), and `prefill_tiles`, runs of up to PREFILL_TILE consecutive tokens of the
    others as (table row, first flat token, count).  The runs with the most keys come first:
    workgroups start in list order, and the last to finish sets the kernel's time."""
    decode_work = [x for row, (start, n, past) in enumerate(zip(shape.q_starts, shape.q_lens, shape.past_lens))
                   if n == 1 for x in (start, past, row, 0)]
    runs = []
    for row, (start, n, past) in enumerate(zip(shape.q_starts, shape.q_lens, shape.past_lens)):
        if n > 1:
            for first in range(0, n, K.PREFILL_TILE):
                count = min(K.PREFILL_TILE, n - first)
                runs.append((past + first + count, (row, start + first, count)))
    runs.sort(key=lambda run: -run[0])
    return {"decode_work": (decode_work, 4), "prefill_tiles": ([x for _, tile in runs for x in tile], 3)}


@register_mixer("attention")
class PagedAttention(Part):
    takes_owed_rows = True

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        if spec.num_heads % spec.num_kv_heads:
            raise ValueError(f"{spec.num_heads} query heads over {spec.num_kv_heads} key/value heads")
        if spec.head_dim % 16 or not 16 <= spec.head_dim <= 256:
            raise ValueError(f"head_dim {spec.head_dim}: the attention kernels take multiples of 16 up to 256")
        self.position = (build_part(POSITION_ENCODINGS, "position encoding", spec.position, dtype, device)
                         if spec.position is not None else
                         POSITION_ENCODINGS["none"](None, dtype, device))

    @property
    def graph_safe(self) -> bool:
        return self.position.graph_safe

    @property
    def graph_max_rows(self):
        return rows_a_graph_may_hold(self.dtype, self.spec.hidden_size, self.spec.num_heads * self.spec.head_dim)

    def decode_fusable(self, rows: int, block_size: int) -> bool:
        """One token a sequence, few rows: the fused projection, the decode attention and the output
        product are all this mixer launches (a rotation that hands out its table runs inside the first)."""
        s = self.spec
        group = s.num_heads // s.num_kv_heads
        return (self.dtype == torch.bfloat16 and 0 < rows <= K.program_max_rows() and self._matrix_cores(block_size)
                and s.head_dim in (64, 128) and group * s.head_dim <= 1024 and not s.out_bias
                and hasattr(self.position, "rotary_table") and s.hidden_size % 8 == 0
                and getattr(s.position, "rotary_dim", 0) % 16 == 0
                and K.program_takes_product(rows, s.hidden_size, K.whole_sum_splits(
                    (s.num_heads + 2 * s.num_kv_heads) * s.head_dim, s.hidden_size, rows))
                and K.program_takes_product(rows, s.num_heads * s.head_dim, K.residual_splits(
                    s.hidden_size, s.num_heads * s.head_dim, rows)))

    def paged_spec(self):
        return attention_pages(self.spec.num_kv_heads, self.spec.head_dim, self.spec.window)

    def _matrix_cores(self, block_size: int) -> bool:
        s = self.spec
        return K.mfma_attention_supported(self.dtype, s.num_heads, s.num_kv_heads, s.head_dim, block_size)

    def step_lists_key(self, block_size: int):
        return WORK_LISTS if self._matrix_cores(block_size) else None

    def step_lists(self, shape: StepShape):
        return attention_work_lists(shape)

    def tensors(self, prefix):
        s = self.spec
        out = {prefix + s.q_name + ".weight": (s.num_heads * s.head_dim, s.hidden_size),
               prefix + s.k_name + ".weight": (s.num_kv_heads * s.head_dim, s.hidden_size),
               prefix + s.v_name + ".weight": (s.num_kv_heads * s.head_dim, s.hidden_size),
               prefix + s.o_name + ".weight": (s.hidden_size, s.num_heads * s.head_dim)}
        if s.qkv_bias:
            out[prefix + s.q_name + ".bias"] = (s.num_heads * s.head_dim,)
            out[prefix + s.k_name + ".bias"] = (s.num_kv_heads * s.head_dim,)
            out[prefix + s.v_name + ".bias"] = (s.num_kv_heads * s.head_dim,)
        if s.out_bias:
            out[prefix + s.o_name + ".bias"] = (s.hidden_size,)
        return out

    def bind(self, prefix, weights):
        s = self.spec
        names = (s.q_name, s.k_name, s.v_name)
        w = torch.cat([weights[prefix + n + ".weight"] for n in names], dim=0)
        b = (torch.cat([weights[prefix + n + ".bias"] for n in names], dim=0) if s.qkv_bias else None)
        self.qkv = Linear(self.matrix(w), None if b is None else self.vector(b))
        nq = s.num_heads * s.head_dim
        self.q_only = Linear(self.qkv.weight[:nq], None if b is None else self.qkv.bias[:nq])
        ob = weights[prefix + s.o_name + ".bias"] if s.out_bias else None
        self.out = Linear(self.matrix(weights[prefix + s.o_name + ".weight"]), None if ob is None else self.vector(ob))

    def _project_encode_store(self, ctx, x, k_cache, v_cache, table):
        """Queries (and, at a stop that owns its cache, keys and values) of the step's tokens:
        projected, encoded by position, the new keys and values stored.  Returns rows whose first
        num_heads * head_dim features are the encoded queries."""
        s = self.spec
        bs = ctx.cache.block_size
        if ctx.writes_cache:
            linear, nkv = self.qkv, s.num_kv_heads
        else:
            linear, nkv, k_cache, v_cache, table = self.q_only, 0, None, None, None
        rotary = getattr(self.position, "rotary_table", None)
        owed = x if isinstance(x, OwedRows) else None
        if owed is not None:
            x = owed.rows
        if rotary is None:
            # any encoding: project, let it encode query and key heads in place, then store
            qkv = linear(owed if owed is not None else x)
            self.position.encode(ctx, qkv, s.num_heads + nkv, s.head_dim)
            if nkv:
                K.kv_store(qkv, s.num_heads, nkv, s.head_dim, ctx.positions, ctx.tok_seq, table, bs, k_cache, v_cache)
            return qkv
        rot, cos_sin = rotary(ctx)
        if x.dtype == torch.bfloat16 and K.skinny_rope_supported(x, linear.weight, s.head_dim, rot):
            # up to 64 rows: one kernel projects, rotates and stores
            q = torch.empty((x.shape[0], s.num_heads * s.head_dim), dtype=x.dtype, device=x.device)
            splits = K.whole_sum_splits(linear.out_features, linear.in_features, x.shape[0])
            K.gemm_skinny_rope(q, x, linear.weight, linear.bias, s.num_heads, nkv, s.head_dim, rot, cos_sin,
                               ctx.positions, ctx.tok_seq, table, bs, k_cache, v_cache, splits,
                               row_scale=owed.row_scale if owed is not None else None)
            return q
        # many rows: the library's plain product (its variant with a bias costs the host six times the
        # call), and the bias is added by the kernel that rotates and stores, which follows anyway
        qkv = linear.without_bias(x) if owed is None else None
        bias = linear.bias if qkv is not None else None
        if qkv is None:
            qkv = linear(owed if owed is not None else x)
        K.rope_kv_write(qkv, s.num_heads, nkv, s.head_dim, rot, cos_sin, ctx.positions, ctx.tok_seq, table, bs,
                        k_cache, v_cache, bias)
        return qkv

    def forward(self, ctx, x):
        """`x`: normalised activations, or `OwedRows` (the projection then pays their scale)."""
        s = self.spec
        pages = ctx.cache.pages_of(ctx.cache_entry)  # as declared in `paged_spec`
        k_cache, v_cache = pages["k"], pages["v"]
        table = ctx.block_tables[ctx.cache.group_of(ctx.cache_entry)]
        qkv = self._project_encode_store(ctx, x, k_cache, v_cache, table)
        attn = torch.empty((x.shape[0], s.num_heads * s.head_dim), dtype=x.dtype, device=x.device)
        geometry = (s.num_heads, s.num_kv_heads, s.head_dim, s.scale, s.window or 0)
        work = ctx.memo.get(WORK_LISTS) if self._matrix_cores(ctx.cache.block_size) else None
        if work is not None:
            decode_work, prefill_tiles = work["decode_work"], work["prefill_tiles"]
            if decode_work.numel():
                K.attn_decode(attn, qkv, k_cache, v_cache, decode_work, table, *geometry)
            if prefill_tiles.numel():
                K.attn_prefill(attn, qkv, k_cache, v_cache, prefill_tiles, ctx.positions, table, *geometry)
        else:
            K.paged_attention_generic(attn, qkv, k_cache, v_cache, ctx.positions, ctx.tok_seq, table, *geometry)
        return self.out.branch(attn, ctx.sink)

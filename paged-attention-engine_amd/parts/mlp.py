"""Dense gated feed-forward: down(silu(gate(x)) * up(x)), no biases
(engine/model.py:317-320 of the reference).  gate and up are one product over
concatenated weights; the gate is applied in float32 and rounded once."""

from __future__ import annotations

import torch

from ..kernels import lib as K
from .base import OwedRows, Part, plain_rows, register_feed_forward
from .linear import Linear, rows_a_graph_may_hold


@register_feed_forward("swiglu")
class SwiGLU(Part):
    graph_safe = True
    takes_owed_rows = True
    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        if spec.activation != "silu":
            raise ValueError(f"activation '{spec.activation}' is not supported by the gated feed-forward")

    @property
    def graph_max_rows(self):
        return rows_a_graph_may_hold(self.dtype, self.spec.hidden_size, self.spec.intermediate_size)

    def tensors(self, prefix):
        s = self.spec
        return {prefix + s.gate_name + ".weight": (s.intermediate_size, s.hidden_size),
                prefix + s.up_name + ".weight": (s.intermediate_size, s.hidden_size),
                prefix + s.down_name + ".weight": (s.hidden_size, s.intermediate_size)}

    BLOCK = 8  # gate and up rows alternate in blocks of this many (the skinny product's gated epilogue)

    def bind(self, prefix, weights):
        s = self.spec
        gate, up = weights[prefix + s.gate_name + ".weight"], weights[prefix + s.up_name + ".weight"]
        inter, hidden = gate.shape
        self.block = self.BLOCK if (self.dtype == torch.bfloat16 and inter % self.BLOCK == 0) else 0
        if self.block:
            b = self.block
            gate_up = torch.stack([gate.view(inter // b, b, hidden), up.view(inter // b, b, hidden)], dim=1)
            gate_up = gate_up.reshape(2 * inter, hidden)
        else:
            gate_up = torch.cat([gate, up], dim=0)
        self.gate_up = Linear(self.matrix(gate_up))
        self.down = Linear(self.matrix(weights[prefix + s.down_name + ".weight"]))

    def decode_fusable(self, rows: int, block_size: int) -> bool:
        s = self.spec
        return (self.dtype == torch.bfloat16 and bool(self.block) and 0 < rows <= K.program_max_rows()
                and s.hidden_size % 8 == 0 and s.intermediate_size % 8 == 0
                and K.program_takes_product(rows, s.hidden_size,
                                            K.whole_sum_splits(2 * s.intermediate_size, s.hidden_size, rows))
                and K.program_takes_product(rows, s.intermediate_size,
                                            K.residual_splits(s.hidden_size, s.intermediate_size, rows)))

    def forward(self, ctx, x):
        """`x`: normalised activations, or `OwedRows` (the gated product then pays their scale)."""
        act = torch.empty((x.shape[0], self.spec.intermediate_size), dtype=x.dtype, device=x.device)
        rows = x.rows if isinstance(x, OwedRows) else x
        if self.block and x.shape[0] and K.skinny_supported(rows, self.gate_up.weight):
            splits = K.whole_sum_splits(2 * self.spec.intermediate_size, self.spec.hidden_size, x.shape[0])
            K.gemm_skinny(act, rows, self.gate_up.weight, None, K.EPI_SWIGLU, splits,
                          row_scale=x.row_scale if isinstance(x, OwedRows) else None)
        else:
            K.swiglu(act, self.gate_up(plain_rows(x)), self.block)
        return self.down.branch(act, getattr(ctx, "sink", None))

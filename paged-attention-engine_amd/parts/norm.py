"""RMS normalisation fused with the pending residual add.

Formula of the reference (engine/model.py:117-123): variance and scaling in
float32, the result cast to the activation type and then multiplied by the
weight.  The residual sum itself stays float32 here (the reference adds in the
activation type, engine/model.py:343,349).
"""

from __future__ import annotations

from typing import Optional

import torch

from ..kernels import lib as K
from .base import OwedRows, Part, ResidualStream, ScaleShape, register_norm


@register_norm("rmsnorm")
class RMSNorm(Part):
    graph_safe = True
    def tensors(self, prefix):
        return {prefix + self.spec.weight_name: ScaleShape((self.spec.size,))}

    def bind(self, prefix, weights):
        self.weight = self.vector(weights[prefix + self.spec.weight_name])

    def folded_for(self, rows: int):
        """(weight, eps) if, in a step of `rows` rows, whatever writes the residual before this norm
        may prepare its rows instead (see `OwedRows`: the consumer's product then pays the scale and
        no norm kernel runs); None if this norm wants to run its own kernel.  The limits are those of
        the products that pay (bfloat16, few rows, rows of 16-byte multiples) and of where it pays
        (`kernels.lib.folds`)."""
        if self.dtype != torch.bfloat16 or not K.folds(rows, self.spec.size) or self.spec.size % 8:
            return None
        return self.weight, self.spec.eps

    def decode_fusable(self, rows: int, block_size: int) -> bool:
        return self.folded_for(rows) is not None  # then `forward` hands prepared rows on and launches nothing

    def forward(self, stream: ResidualStream, rows: Optional[torch.Tensor] = None):
        """Add the pending branch output into the residual and return the normalised
        rows.  With `rows` (int32 indices) only those rows are produced and the
        stream is left untouched.  When the branch before has added itself into the residual
        and prepared this norm's rows, they are returned as they are (`OwedRows`): no kernel runs."""
        if stream.owed is not None:
            owed, mine = stream.owed, stream.owed_to is self
            if rows is None:
                stream.owed = stream.owed_to = None
                if mine:
                    return owed
            # prepared for another norm, or only some rows are wanted: the residual is complete
        n = stream.residual.shape[0] if rows is None else rows.numel()
        out = torch.empty((n, self.spec.size), dtype=self.dtype, device=stream.residual.device)
        K.add_rmsnorm(stream.residual, stream.pending, self.weight, self.spec.eps, out, rows)
        if rows is None:
            stream.pending = None
        return out

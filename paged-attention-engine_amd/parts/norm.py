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
from .base import OwedRows, Part, ResidualStream, register_norm


@register_norm("rmsnorm")
class RMSNorm(Part):
    graph_safe = True
    def tensors(self, prefix):
        return {prefix + "weight": (self.spec.size,)}

    def bind(self, prefix, weights):
        self.weight = self.vector(weights[prefix + "weight"])

    def folded(self):
        """(weight, eps): what a product needs to prepare rows for this norm (see `OwedRows`)."""
        return self.weight, self.spec.eps

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

"""y = x W^T + b, the matrix product every part shares.

The reference calls F.linear on weights stored (out_features, in_features)
(engine/model.py:303-305,315,318-320).  In float32 this engine runs its own
product kernel, which accumulates in float32 in k order with no reduced
precision; in bfloat16 large products go to the platform's matrix library (as
the reference's go to its library) and accumulate in float32.
"""

from __future__ import annotations

from typing import Optional

import torch

from ..kernels import lib as K


class Linear:
    def __init__(self, weight: torch.Tensor, bias: Optional[torch.Tensor] = None) -> None:
        assert weight.dim() == 2 and weight.is_contiguous()
        self.weight = weight
        self.bias = bias
        self.out_features, self.in_features = weight.shape

    def __call__(self, x: torch.Tensor, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        out_dtype = out_dtype or x.dtype
        out = torch.empty((x.shape[0], self.out_features), dtype=out_dtype, device=x.device)
        if x.shape[0] == 0:
            return out
        if x.dtype == torch.float32 or out_dtype != x.dtype:
            K.gemm_plain(out, x, self.weight, self.bias)
        else:
            bias = self.bias
            if bias is not None and bias.dtype != x.dtype:
                bias = bias.to(x.dtype)
            if bias is None:
                torch.mm(x, self.weight.t(), out=out)
            else:
                torch.addmm(bias, x, self.weight.t(), out=out)
        return out

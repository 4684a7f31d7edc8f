"""y = x W^T + b, the matrix product every part shares.

The reference calls F.linear on weights stored (out_features, in_features)
(engine/model.py:303-305,315,318-320).  Here:

  float32    this engine's own product kernel: float32 fused multiply-adds in k
             order, no reduced-precision matrix mode, each row independent of the
             batch;
  bfloat16   up to 64 rows (decode steps, small portions): the weight-streaming
             matrix-core kernel, which reads W once; more rows: the platform's
             matrix library, as the reference's products go to its library.
             Both accumulate in float32.
"""

from __future__ import annotations

from typing import Optional

import torch

from ..kernels import lib as K
from .base import OwedRows


def rows_a_graph_may_hold(dtype: torch.dtype, *inner_sizes: int):
    """For products with these inner sizes: up to how many rows every one of them runs in this
    engine's own kernels, which is what recording a step as a HIP graph needs (library products
    may record memory clears into a graph).  None: any number of rows; 0: never."""
    if dtype == torch.float32:
        return None
    return K.SKINNY_MAX_ROWS if all(size % 8 == 0 for size in inner_sizes) else 0


class Linear:
    def __init__(self, weight: torch.Tensor, bias: Optional[torch.Tensor] = None) -> None:
        assert weight.dim() == 2 and weight.is_contiguous()
        self.weight = weight
        self.bias = bias
        self.out_features, self.in_features = weight.shape

    @property
    def graph_max_rows(self):
        return rows_a_graph_may_hold(self.weight.dtype, self.in_features)

    def _library(self, x: torch.Tensor, with_bias: bool = True) -> torch.Tensor:
        out = torch.empty((x.shape[0], self.out_features), dtype=x.dtype, device=x.device)
        bias = self.bias if with_bias else None
        if bias is None:
            torch.mm(x, self.weight.t(), out=out)
        else:
            torch.addmm(bias if bias.dtype == x.dtype else bias.to(x.dtype), x, self.weight.t(), out=out)
        return out

    def __call__(self, x) -> torch.Tensor:
        """[M, N] in x's dtype.  `x` may be `OwedRows`: the few-row product pays their scale itself."""
        if isinstance(x, OwedRows):
            if x.shape[0] and K.skinny_supported(x.rows, self.weight):
                out = torch.empty((x.shape[0], self.out_features), dtype=x.dtype, device=x.device)
                K.gemm_skinny(out, x.rows, self.weight, self.bias, K.EPI_BF16, row_scale=x.row_scale)
                return out
            x = x.settle()
        M = x.shape[0]
        if x.dtype == torch.float32 or M == 0:
            out = torch.empty((M, self.out_features), dtype=x.dtype, device=x.device)
            if M:
                K.gemm_plain(out, x, self.weight, self.bias)
            return out
        if K.skinny_supported(x, self.weight):
            out = torch.empty((M, self.out_features), dtype=x.dtype, device=x.device)
            K.gemm_skinny(out, x, self.weight, self.bias, K.EPI_BF16)
            return out
        return self._library(x)

    def without_bias(self, x) -> Optional[torch.Tensor]:
        """The product without its bias where that is the cheaper call (the matrix library's plain
        product, many rows), for a caller that adds the bias in a kernel of its own that follows
        anyway; None where the bias costs nothing (this engine's own products)."""
        if (self.bias is None or isinstance(x, OwedRows) or x.dtype != torch.bfloat16 or x.shape[0] == 0
                or K.skinny_supported(x, self.weight)):
            return None
        return self._library(x, with_bias=False)

    def branch(self, x: torch.Tensor, sink=None) -> Optional[torch.Tensor]:
        """The product as a residual branch's output: [M, N] in x's dtype, or float32
        partial sums [P, M, N] that the next norm adds up in order (no bias then).  With a `sink`
        whose norm can be folded, the few-row product adds itself into the residual instead and
        prepares the following product's rows; nothing is returned then."""
        if x.dtype == torch.bfloat16 and self.bias is None and x.shape[0] and K.skinny_supported(x, self.weight):
            splits = K.skinny_splits(self.out_features, self.in_features, x.shape[0])
            fold = sink.folded(x.shape[0]) if sink is not None else None
            residual = sink.stream.residual if sink is not None else None
            if (fold is not None and residual.dtype == torch.float32
                    and residual.is_contiguous() and tuple(residual.shape) == (x.shape[0], self.out_features)):
                weight, eps = fold
                rows = torch.empty((x.shape[0], self.out_features), dtype=torch.bfloat16, device=x.device)
                stats = torch.empty((x.shape[0], K.stat_tiles(self.out_features)), dtype=torch.float32, device=x.device)
                K.gemm_skinny(residual, x, self.weight, None, K.EPI_RESIDUAL,
                              K.residual_splits(self.out_features, self.in_features, x.shape[0]),
                              following=(rows, weight, stats))
                sink.deliver(OwedRows(rows, stats, eps))
                return None
            out = torch.empty((splits, x.shape[0], self.out_features), dtype=torch.float32, device=x.device)
            K.gemm_skinny(out, x, self.weight, None, K.EPI_F32, splits)
            return out
        return self(x)

    def float32(self, x: torch.Tensor) -> torch.Tensor:
        """[M, N] float32 whatever x's dtype (the head's logits)."""
        M = x.shape[0]
        out = torch.empty((M, self.out_features), dtype=torch.float32, device=x.device)
        if M == 0:
            return out
        if x.dtype == torch.float32:
            K.gemm_plain(out, x, self.weight, self.bias)
        elif x.shape[1] % 8 == 0:
            for first in range(0, M, K.SKINNY_MAX_ROWS):
                rows = slice(first, min(M, first + K.SKINNY_MAX_ROWS))
                K.gemm_skinny(out[rows], x[rows], self.weight, self.bias, K.EPI_F32)
        else:
            K.gemm_plain(out, x, self.weight, self.bias)
        return out

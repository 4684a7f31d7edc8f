"""Choosing the next token: greedy, or by temperature with a reproducible draw.

The reference samples greedily only: `int(torch.argmax(logits).item())` per
sequence per step (engine/scheduler.py:610, engine/model.py:491), the first
maximum winning ties.  Temperature sampling is this engine's own: the token is
the first index whose cumulative probability under softmax(logits / T) exceeds
u * total, where u in [0, 1) is a function of (seed, request id, index of the
generated token) alone, so a request draws the same tokens whatever else is in
the batch and however its prompt was cut.  Both run in one kernel over the
float32 logits, and one copy brings all of a step's tokens to the host.
"""

from __future__ import annotations

import zlib
from typing import Optional, Sequence

import torch

from ..kernels import lib as K

_MASK = (1 << 64) - 1


def _splitmix64(x: int) -> int:
    x = (x + 0x9E3779B97F4A7C15) & _MASK
    x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & _MASK
    return x ^ (x >> 31)


def uniform_for(seed: int, request_id: str, index: int) -> float:
    """The draw of generated token `index` of a request: 24 bits, so it is exact in float32."""
    key = _splitmix64((int(seed) & _MASK) ^ (zlib.crc32(request_id.encode("utf-8")) << 32))
    return (_splitmix64(key ^ (index & _MASK)) >> 40) / float(1 << 24)


class SampledTokens:
    """A step's tokens, sampled on the device and on their way to the host."""

    def __init__(self, on_device: torch.Tensor) -> None:
        self.on_device = on_device  # int32 [R]; what the next step may be fed from
        self._host = torch.empty(on_device.shape, dtype=torch.int32, pin_memory=True)
        self._host.copy_(on_device, non_blocking=True)
        self._arrived = torch.cuda.Event()
        self._arrived.record()

    def wait(self) -> list:
        self._arrived.synchronize()
        return self._host.tolist()


class Sampler:
    def __init__(self, device) -> None:
        self.device = device

    def sample_on_device(self, logits: torch.Tensor, temperatures: Sequence[float],
                         uniforms: Sequence[float]) -> SampledTokens:
        """As `sample`, without waiting: the tokens stay on the device for the next step and
        come to the host behind an event."""
        rows = logits.shape[0]
        tokens = torch.empty(rows, dtype=torch.int32, device=logits.device)
        if rows:
            if any(t > 0 for t in temperatures):
                params = torch.tensor([list(temperatures), list(uniforms)], dtype=torch.float32).to(
                    logits.device, non_blocking=True)
                K.sample(tokens, logits, params[0], params[1])
            else:
                K.sample(tokens, logits, None, None)
        return SampledTokens(tokens)

    def sample(self, logits: torch.Tensor, temperatures: Sequence[float],
               uniforms: Sequence[float]) -> list:
        """Tokens for the rows of `logits` (float32 [R, V] on the GPU)."""
        rows = logits.shape[0]
        if rows == 0:
            return []
        tokens = torch.empty(rows, dtype=torch.int32, device=logits.device)
        if any(t > 0 for t in temperatures):
            params = torch.tensor([list(temperatures), list(uniforms)], dtype=torch.float32).to(logits.device)
            K.sample(tokens, logits, params[0], params[1])
        else:
            K.sample(tokens, logits, None, None)
        return tokens.cpu().tolist()

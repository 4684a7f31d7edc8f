"""Arrangements of a layer's parts.

"prenorm" is the reference's block (engine/model.py:340-349):
h = h + mixer(norm1(h)); h = h + feed_forward(norm2(h)).  Each branch's output is
left pending on the stream and added by the next norm, in float32.
"""

from __future__ import annotations

from .base import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, BranchSink, Part, ResidualStream, build_part, plain_rows,
                   register_block)


@register_block("prenorm")
class PreNormBlock:
    def __init__(self, layer_spec, dtype, device):
        self.spec = layer_spec
        self.mixer_norm = build_part(NORMS, "norm", layer_spec.mixer_norm, dtype, device)
        self.mixer = build_part(MIXERS, "mixer", layer_spec.mixer, dtype, device)
        self.feed_forward_norm = build_part(NORMS, "norm", layer_spec.feed_forward_norm, dtype, device)
        self.feed_forward = build_part(FEED_FORWARDS, "feed-forward", layer_spec.feed_forward, dtype, device)

    @property
    def graph_safe(self) -> bool:
        return all(part.graph_safe for part, _ in self._named())

    @property
    def graph_max_rows(self):
        """The fewest rows any part allows a recorded step to hold (None: no part sets a limit)."""
        limits = [part.graph_max_rows for part, _ in self._named() if part.graph_max_rows is not None]
        return min(limits) if limits else None

    def parts(self):
        return [part for part, _ in self._named()]

    def _named(self):
        s = self.spec
        return ((self.mixer_norm, s.prefix + s.mixer_norm_prefix), (self.mixer, s.prefix + s.mixer_prefix),
                (self.feed_forward_norm, s.prefix + s.feed_forward_norm_prefix),
                (self.feed_forward, s.prefix + s.feed_forward_prefix))

    def tensors(self):
        out = {}
        for part, prefix in self._named():
            out.update(part.tensors(prefix))
        return out

    def bind(self, weights):
        for part, prefix in self._named():
            part.bind(prefix, weights)

    def decode_fusable(self, rows: int, block_size: int) -> bool:
        """Whether a step of `rows` single tokens runs this block through recordable kernels alone."""
        return all(part.decode_fusable(rows, block_size) for part, _ in self._named())

    def entry_fold(self, rows: int):
        """(norm, weight, eps) if whatever fills the stream before this block (the embedding) may
        prepare the first norm's rows for a step of `rows` rows; None if the norm runs its own kernel."""
        fold = getattr(self.mixer_norm, "folded_for", None) if self.mixer.takes_owed_rows else None
        got = fold(rows) if fold is not None else None
        return None if got is None else (self.mixer_norm, *got)

    def forward(self, ctx, stream: ResidualStream) -> None:
        """Each branch is offered a sink: its last product may add itself into the residual and
        prepare the rows of the norm that reads the stream next (this block's second norm, then
        `stream.next_norm`, the first norm of the block that follows), which then runs no kernel."""
        x = self.mixer_norm.forward(stream)
        ctx.sink = BranchSink(stream, self.feed_forward_norm)
        stream.pending = self.mixer.forward(ctx, x if self.mixer.takes_owed_rows else plain_rows(x))
        x = self.feed_forward_norm.forward(stream)
        ctx.sink = BranchSink(stream, stream.next_norm) if stream.next_norm is not None else None
        stream.pending = self.feed_forward.forward(ctx, x if self.feed_forward.takes_owed_rows else plain_rows(x))
        ctx.sink = None


def build_block(layer_spec, dtype, device):
    if layer_spec.arrangement not in BLOCKS:
        raise KeyError(f"no block arrangement '{layer_spec.arrangement}'; known: {', '.join(sorted(BLOCKS))}")
    return BLOCKS[layer_spec.arrangement](layer_spec, dtype, device)

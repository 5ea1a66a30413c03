"""Pre-norm residual block: h += mixer(norm(h)); h += feed_forward(norm(h))
(src/models/qwen2/graph.rs:59-177 of yusiwen/minfer).  When only some rows are wanted after
this block (the last one of a step), they are gathered between the two halves, so the
feed-forward runs on those rows only, as the reference does for its tail rows
(graph.rs:126-138)."""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import Block, announce_norm, normed_input, register_block


@register_block("prenorm")
class PreNormBlock(Block):
    """norms: "mixer" before the mixer, "feed_forward" before the feed-forward.  A block without a
    mixer or without a feed-forward (and then without that branch's norm) is that branch left out."""

    needs_mixer = False
    needs_feed_forward = False
    norm_names = ()
    optional_norms = ("mixer", "feed_forward")

    def __init__(self, mixer, feed_forward, norms, rt):
        super().__init__(mixer, feed_forward, norms, rt)
        for part, name in ((mixer, "mixer"), (feed_forward, "feed_forward")):
            if (part is None) != (name not in self.norms):
                raise ValueError(f"prenorm block: the {name} and the norm before it come together or not at all")

    def first_norm(self):
        return self.mixer_norm if self.mixer is not None else self.feed_forward_norm

    def forward(self, h, ctx, entry: int, writes_cache: bool, keep_rows=None):
        after = getattr(ctx, "norm_after_block", None)      # the norm that reads the stream behind this block
        if self.mixer is not None:
            x = normed_input(self.mixer_norm, self.mixer, h, ctx=ctx)
            # the mixer's output meets the feed-forward's norm, unless rows are dropped in between
            announce_norm(ctx, (self.feed_forward_norm if self.feed_forward is not None else after)
                          if keep_rows is None else None)
            self.mixer.forward(x, h, ctx, entry, writes_cache)
            ctx.norm_next = None
        if keep_rows is not None:
            kept = torch.empty((keep_rows.numel(), h.shape[1]), dtype=h.dtype, device=h.device)
            ops.gather_rows(h, keep_rows, kept)
            h = kept
        if self.feed_forward is not None:
            x = normed_input(self.feed_forward_norm, self.feed_forward, h, ctx=ctx)
            announce_norm(ctx, after)
            self.feed_forward.forward(x, h, ctx)
            ctx.norm_next = None
        return h

"""Pre-norm residual block: h += mixer(norm(h)); h += feed_forward(norm(h))
(src/models/qwen2/graph.rs:59-177 of yusiwen/minfer).  When only some rows are wanted after
this block (the last one of a step), they are gathered between the two halves, so the
feed-forward runs on those rows only, as the reference does for its tail rows
(graph.rs:126-138)."""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import Block, normed_input, register_block


@register_block("prenorm")
class PreNormBlock(Block):
    def forward(self, h, ctx, entry: int, writes_cache: bool, keep_rows=None):
        x = normed_input(self.mixer_norm, self.mixer, h)
        self.mixer.forward(x, h, ctx, entry, writes_cache)
        if keep_rows is not None:
            kept = torch.empty((keep_rows.numel(), h.shape[1]), dtype=h.dtype, device=h.device)
            ops.gather_rows(h, keep_rows, kept)
            h = kept
        x = normed_input(self.feed_forward_norm, self.feed_forward, h)
        self.feed_forward.forward(x, h, ctx)
        return h

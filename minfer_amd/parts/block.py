"""Pre-norm residual block: h += mixer(norm(h)); h += feed_forward(norm(h))
(src/models/qwen2/graph.rs:59-177 of yusiwen/minfer).  When only some rows are wanted after
this block (the last one of a step), they are gathered between the two halves, so the
feed-forward runs on those rows only, as the reference does for its tail rows
(graph.rs:126-138)."""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import Block, register_block


@register_block("prenorm")
class PreNormBlock(Block):
    def forward(self, h, ctx, entry: int, writes_cache: bool, keep_rows=None):
        x = self.mixer_norm.forward(h)
        self.mixer.forward(x, h, ctx, entry, writes_cache)
        if keep_rows is not None:
            kept = torch.empty((keep_rows.numel(), h.shape[1]), dtype=h.dtype, device=h.device)
            ops.gather_rows(h, keep_rows, kept)
            h = kept
        x = self.feed_forward_norm.forward(h)
        self.feed_forward.forward(x, h, ctx)
        return h

"""SwiGLU feed-forward without biases: down( silu(gate x) * (up x) ), silu(z) = z/(1+e^-z)
(src/models/qwen2/graph.rs:154-176, src/graph/cpu_backend.rs:323-329 of yusiwen/minfer).
gate|up are one matrix.  In bfloat16 its rows are interleaved so that the product's epilogue
applies SwiGLU from the 32-bit accumulators and writes y directly; in 32-bit the stacked
product is followed by the SwiGLU kernel.  The down product adds into the residual."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.loader import TensorSpec
from .base import FeedForward, Normed, register_feed_forward
from .linear import Linear


@register_feed_forward("swiglu")
class SwiGLU(FeedForward):
    """params: hidden_size, intermediate_size, gate/up/down (tensor name stems)."""

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        p = spec.params
        self.hidden, self.inter = int(p["hidden_size"]), int(p["intermediate_size"])
        self.names = {k: p[k] for k in ("gate", "up", "down")}
        self.gate_up = self.down = self.fused = self.fused_tiled = None

    def tensor_specs(self):
        n = self.names
        return {n["gate"] + ".weight": TensorSpec((self.inter, self.hidden)),
                n["up"] + ".weight": TensorSpec((self.inter, self.hidden)),
                n["down"] + ".weight": TensorSpec((self.hidden, self.inter))}

    def load(self, get):
        n = self.names
        gate, up = get(n["gate"] + ".weight"), get(n["up"] + ".weight")
        if self.rt.is_bf16 and gate.dtype == up.dtype == torch.bfloat16:
            self.fused = ops.interleave_gate_up(gate, up)
        else:
            self.gate_up = Linear.stacked([gate, up])
        self.down = Linear(get(n["down"] + ".weight"))

    def decode_copies(self, make: bool, min_row_length: int = 0) -> int:
        n = self.down.decode_copy(make, min_row_length)
        if self.fused is not None:
            if self.hidden % 32 == 0 and self.hidden >= min_row_length:
                if make and self.fused_tiled is None:
                    self.fused_tiled = ops.tile_weight(self.fused)
                n += self.fused.numel() * 2
        elif self.gate_up is not None:
            n += self.gate_up.decode_copy(make, min_row_length)
        return n

    takes_normed = True

    def forward(self, x, h, ctx) -> None:
        y = torch.empty((x.shape[0], self.inter), dtype=self.rt.dtype, device=x.device)
        if self.fused is not None:
            fold = x.norm.rms_scale() if isinstance(x, Normed) else None
            done = False
            if fold is not None and x.ahead is not None:      # the product before prepared this norm's input
                done = ops.linear_fused(x.ahead.xg, self.fused, None, y, tiled=self.fused_tiled, swiglu=True,
                                        scale_in=(x.ahead.sums, fold[1]))
            if not done and fold is not None:
                done = ops.linear_normed(x.h, fold[0], fold[1], x.row_idx, self.fused, None, y, swiglu=True,
                                         tiled=self.fused_tiled)
            if not done:
                ops.linear_swiglu(x.tensor() if isinstance(x, Normed) else x, self.fused, y, tiled=self.fused_tiled)
        else:
            ops.swiglu(self.gate_up(x, out_dtype=torch.float32), y)
        self.down(y, out=h, accumulate=True, ctx=ctx)

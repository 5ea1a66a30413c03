"""SwiGLU feed-forward without biases: down( silu(gate x) * (up x) ), silu(z) = z/(1+e^-z)
(src/models/qwen2/graph.rs:154-176, src/graph/cpu_backend.rs:323-329 of yusiwen/minfer).
gate|up are one stacked matrix; the down product adds into the residual."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.loader import TensorSpec
from .base import FeedForward, register_feed_forward
from .linear import Linear


@register_feed_forward("swiglu")
class SwiGLU(FeedForward):
    """params: hidden_size, intermediate_size, gate/up/down (tensor name stems)."""

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        p = spec.params
        self.hidden, self.inter = int(p["hidden_size"]), int(p["intermediate_size"])
        self.names = {k: p[k] for k in ("gate", "up", "down")}
        self.gate_up = self.down = None

    def tensor_specs(self):
        n = self.names
        return {n["gate"] + ".weight": TensorSpec((self.inter, self.hidden)),
                n["up"] + ".weight": TensorSpec((self.inter, self.hidden)),
                n["down"] + ".weight": TensorSpec((self.hidden, self.inter))}

    def load(self, get):
        n = self.names
        self.gate_up = Linear.stacked([get(n["gate"] + ".weight"), get(n["up"] + ".weight")])
        self.down = Linear(get(n["down"] + ".weight"))

    def forward(self, x, h, ctx) -> None:
        gu = self.gate_up(x, out_dtype=torch.float32)
        y = torch.empty((x.shape[0], self.inter), dtype=self.rt.dtype, device=x.device)
        ops.swiglu(gu, y)
        self.down(y, out=h, accumulate=True)

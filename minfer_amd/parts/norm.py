"""RMSNorm: y = x / sqrt(mean(x^2) + eps) * w, eps inside the root (src/vec_ops.rs:500-522
of yusiwen/minfer; the three places it stands in the layer, src/models/qwen2/graph.rs:63,
155,180).  Statistics in 32-bit over the float32 residual stream."""
from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops
from ..weights.loader import TensorSpec
from .base import Norm, register_norm


@register_norm("rmsnorm")
class RMSNorm(Norm):
    """params: size, eps, weight (tensor name)."""

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.size, self.eps, self.name = int(spec.params["size"]), float(spec.params["eps"]), spec.params["weight"]
        self.weight = None

    def tensor_specs(self):
        return {self.name: TensorSpec((self.size,), init="ones")}

    def load(self, get):
        self.weight = get(self.name).to(torch.float32).contiguous()

    def rms_scale(self):
        return self.weight, self.eps

    def forward(self, h, out: Optional[torch.Tensor] = None, row_idx: Optional[torch.Tensor] = None):
        rows = h.shape[0] if row_idx is None else row_idx.numel()
        if out is None:
            out = torch.empty((rows, self.size), dtype=self.rt.dtype, device=h.device)
        ops.rmsnorm(h, self.weight, self.eps, out, row_idx)
        return out

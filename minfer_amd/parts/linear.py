"""A weight matrix `[out][in]` with an optional bias, applied through the HIP products.

out[t][o] = dot(W[o][:], x[t][:]) + b[o] (src/graph/cpu_backend.rs:214-248 of
yusiwen/minfer).  A matrix stored in 32 bits stays in 32 bits and takes the 32-bit kernel
even when activations are bfloat16 (they are widened, which is exact).  Biases are kept in
float32 and added in the product's epilogue.
"""
from __future__ import annotations

from typing import List, Optional

import torch

from ..kernels import ops, tuning
from .base import NormAhead, Normed


def common_matrix_dtype(tensors: List[torch.Tensor]) -> torch.dtype:
    return torch.bfloat16 if all(t.dtype == torch.bfloat16 for t in tensors) else torch.float32


class Linear:
    def __init__(self, weight: torch.Tensor, bias: Optional[torch.Tensor] = None):
        if weight.dim() != 2:
            raise ValueError(f"Linear: weight must be a matrix, got {tuple(weight.shape)}")
        self.weight = weight.contiguous()
        self.bias = None if bias is None else bias.to(torch.float32).contiguous()
        self.out_features, self.in_features = weight.shape
        self.tiled: Optional[torch.Tensor] = None      # ops.tile_weight(weight), where the model keeps one

    def decode_copy(self, make: bool, min_row_length: int = 0) -> int:
        """Bytes of the tiled copy of this matrix, which the products of few rows read faster than
        the matrix itself (0: it has none: 32-bit, a row length that is no multiple of 32, or a
        row shorter than `min_row_length`: the long rows gain most); made when `make`."""
        if self.weight.dtype != torch.bfloat16 or self.in_features % 32 or self.in_features < min_row_length:
            return 0
        if make and self.tiled is None:
            self.tiled = ops.tile_weight(self.weight)
        return (self.out_features + 15) // 16 * 16 * self.in_features * 2

    @classmethod
    def stacked(cls, weights: List[torch.Tensor], biases: Optional[List[Optional[torch.Tensor]]] = None):
        """Rows of several matrices over the same input in one matrix, so a step reads one
        (the reference concatenates q|k|v and gate|up the same way for its GPU path,
        src/models/qwen2/loader.rs:290-331)."""
        dt = common_matrix_dtype(weights)
        w = torch.cat([t.to(dt) for t in weights], dim=0)
        b = None
        if biases is not None and any(x is not None for x in biases):
            b = torch.cat([torch.zeros(t.shape[0], dtype=torch.float32, device=t.device) if x is None
                           else x.to(torch.float32) for t, x in zip(weights, biases)])
        return cls(w, b)

    def __call__(self, x, out: Optional[torch.Tensor] = None,
                 out_dtype: torch.dtype = torch.float32, accumulate: bool = False, ctx=None) -> torch.Tensor:
        """`ctx`: the step's context, from a part whose output this product adds into the residual
        stream: where the block has announced the norm that reads the stream next, the product
        may prepare that norm's input on its way out (`_prepare_norm`)."""
        rows = x.shape[0]
        if out is None:
            out = torch.empty((rows, self.out_features), dtype=out_dtype, device=x.device)
        if isinstance(x, Normed):
            if self.weight.dtype == torch.bfloat16:
                if x.ahead is not None and ops.linear_fused(x.ahead.xg, self.weight, self.bias, out, accumulate=accumulate,
                                                            tiled=self.tiled, scale_in=(x.ahead.sums, x.norm.rms_scale()[1])):
                    return out
                fold = x.norm.rms_scale()
                if fold is not None and ops.linear_normed(x.h, fold[0], fold[1], x.row_idx, self.weight, self.bias,
                                                          out, accumulate=accumulate, tiled=self.tiled):
                    return out
            x = x.tensor()
        if self.weight.dtype == torch.float32 and x.dtype != torch.float32:
            wide = torch.empty(x.shape, dtype=torch.float32, device=x.device)
            ops.convert(x, wide)
            x = wide
        if x.dtype == torch.float32 and out.dtype != torch.float32:
            tmp = torch.empty(out.shape, dtype=torch.float32, device=x.device)
            ops.linear(x, self.weight, self.bias, tmp)
            ops.convert(tmp, out)
            return out
        if ctx is not None and self._prepare_norm(x, out, accumulate, ctx):
            return out
        ops.linear(x, self.weight, self.bias, out, accumulate=accumulate, tiled=self.tiled)
        return out

    def _prepare_norm(self, x: torch.Tensor, out: torch.Tensor, accumulate: bool, ctx) -> bool:
        """Runs the product with the next norm's input prepared beside it (bf16(out g) and the rows'
        partial sums of squares, left in `ctx.norm_ahead`) where the block has said which norm
        that is, the norm is of the RMS form and the product's kernels have a place for it (steps of
        17 to 64 rows whose K is split over blocks; steps of at most 16 rows in the one-kernel
        forms).  False: nothing ran."""
        norm = getattr(ctx, "norm_next", None)
        if norm is None or not 0 < x.shape[0] <= 64 or x.dtype != torch.bfloat16 or out.dtype != torch.float32:
            return False
        if tuning.NO_NORM_AHEAD or x.device.type != "cuda":
            return False
        lo, hi = ops.NORM_AHEAD_16_WIDTHS
        if x.shape[0] <= 16 and not lo <= self.out_features <= hi:
            return False
        fold = norm.rms_scale()
        if fold is None or fold[0].numel() != self.out_features:
            return False
        xg = torch.empty(out.shape, dtype=torch.bfloat16, device=out.device)
        sums = torch.empty((out.shape[0], ops.norm_sum_parts(self.out_features, out.shape[0])), dtype=torch.float32,
                           device=out.device)
        if not ops.linear_fused(x, self.weight, self.bias, out, accumulate=accumulate, tiled=self.tiled,
                                norm_out=(fold[0], xg, sums)):
            return False
        ctx.norm_ahead = NormAhead(norm, out, xg, sums)
        return True

"""The sampling pipeline on the device, in the reference's order: penalties -> greedy if
temperature < 1e-6 -> top-k -> top-p -> temperature draw (`sample_with_penalties`,
src/sampler.rs:272-290 of yusiwen/minfer).  Logits are changed in place (a small top-k takes one
fused kernel for the last three steps, which leaves them alone)."""
from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops
from .params import SamplingParams
from .rng import stream_i64


class Sampler:
    def __init__(self, params: SamplingParams):
        params.validate()
        self.params = params

    def streams(self, keys) -> list:
        """The random stream ids (int64 values) of the sequences with these keys under the
        sampler's seed: what `__call__` takes as `streams`."""
        return [stream_i64(self.params.seed, int(k)) for k in keys]

    @property
    def structure(self):
        """What of the options shapes the kernels that run (the seed does not: it is data)."""
        from dataclasses import replace
        return replace(self.params, seed=0)

    def __call__(self, logits: torch.Tensor, streams: torch.Tensor, steps: torch.Tensor, out: torch.Tensor,
                 prev: Optional[torch.Tensor] = None, n_prev: Optional[torch.Tensor] = None) -> torch.Tensor:
        """logits float32 [rows][vocab]; streams int64 [rows] (`streams(keys)`, one per sequence);
        steps int32 [rows] (draws made so far); prev int32 [rows][window] and n_prev int32 [rows]
        hold each sequence's recent tokens when penalties are on.  Writes token ids into `out`
        (int32)."""
        p = self.params
        if p.has_penalties:
            if prev is None or n_prev is None:
                raise ValueError("penalties need the recent-token window")
            ops.penalties(logits, prev, n_prev, p.repeat_penalty, p.frequency_penalty, p.presence_penalty)
        if p.is_greedy:
            ops.argmax(logits, out)
            return out
        if ops.sample_filtered_takes(logits.shape[-1], p.top_k, p.temp):
            ops.sample_filtered(logits, p.top_k, p.top_p, p.temp, streams, steps, out)
            return out
        if p.top_k > 0:
            ops.top_k(logits, p.top_k)
        if 0.0 < p.top_p < 1.0:
            ops.top_p(logits, p.top_p)
        ops.sample(logits, p.temp, streams, steps, out)
        return out

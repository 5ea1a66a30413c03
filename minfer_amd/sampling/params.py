"""Sampling options with the reference's names, meanings and defaults (`GenParams`,
src/main.rs:42-70 of yusiwen/minfer): temperature 0.8 (below 1e-6 means greedy), top-k 40
(0 = off), top-p 0.95 (<= 0 or >= 1 = off), repeat penalty 1.1 (1 = off), frequency and
presence penalties 0, a window of the last 64 tokens for the penalties (src/main.rs:539),
seed 42."""
from __future__ import annotations

from dataclasses import dataclass

REPEAT_LAST_N = 64


@dataclass(frozen=True)
class SamplingParams:
    temp: float = 0.8
    top_k: int = 40
    top_p: float = 0.95
    repeat_penalty: float = 1.1
    frequency_penalty: float = 0.0
    presence_penalty: float = 0.0
    seed: int = 42

    @classmethod
    def greedy(cls, **kw) -> "SamplingParams":
        """Plain argmax: temperature 0 and no penalties."""
        base = dict(temp=0.0, top_k=0, top_p=1.0, repeat_penalty=1.0)
        base.update(kw)
        return cls(**base)

    @property
    def is_greedy(self) -> bool:
        return self.temp < 1e-6

    @property
    def has_penalties(self) -> bool:
        return (abs(self.repeat_penalty - 1.0) >= 1e-6 or abs(self.frequency_penalty) >= 1e-6
                or abs(self.presence_penalty) >= 1e-6)

    def validate(self) -> None:
        if self.temp < 0:
            raise ValueError(f"temp must be >= 0, got {self.temp}")
        if self.top_k < 0:
            raise ValueError(f"top_k must be >= 0, got {self.top_k}")

"""Descriptions of a model as data: which parts make up each block, with which constants,
and in which order blocks run.

A configuration class turns its config.json keys into a `ModelSpec`; the builder in
`minfer_amd.engine.model` turns a `ModelSpec` into parts by looking each `PartSpec.kind`
up in the part registries.  No part ever sees the configuration or the model it is in.

The reference builds its per-step graph from part constructors that take their constants
as parameters (`rms_norm(x,w,eps)`, `rope(x,pos,style,meta)`, `attn(q,kv,pos,mode,meta)`,
src/graph/builder.rs:79-286 of yusiwen/minfer) inside one loop over layers
(src/models/qwen2/graph.rs:59-177).  Here that loop is the `schedule` list.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, Mapping, Optional, Tuple


@dataclass(frozen=True)
class PartSpec:
    """One part: its registry name and its constants (sizes, eps, theta, tensor names...)."""
    kind: str
    params: Dict[str, Any] = field(default_factory=dict)

    def get(self, key: str, default: Any = None) -> Any:
        return self.params.get(key, default)


@dataclass(frozen=True)
class BlockSpec:
    """One block: the arrangement (`kind`, e.g. pre-norm residual), its mixer and feed-forward
    (either may be absent) and its norms by the names the arrangement gives them.  `prefix` is
    put before every tensor name of the block's parts.  `mixer_norm` and `feed_forward_norm` are
    short for the norms named "mixer" and "feed_forward", the two that a pre-norm block has; an
    arrangement with others (a norm after each branch as well, one norm shared by two parallel
    branches) names them in `norms`."""
    kind: str
    prefix: str
    mixer: Optional[PartSpec] = None
    feed_forward: Optional[PartSpec] = None
    mixer_norm: Optional[PartSpec] = None
    feed_forward_norm: Optional[PartSpec] = None
    norms: Mapping[str, PartSpec] = field(default_factory=dict)

    def __post_init__(self):
        norms = dict(self.norms)
        for name, short in (("mixer", self.mixer_norm), ("feed_forward", self.feed_forward_norm)):
            if short is not None:
                if name in norms and norms[name] != short:
                    raise ValueError(f"block {self.prefix!r}: the norm {name!r} is given twice")
                norms[name] = short
        object.__setattr__(self, "norms", norms)
        object.__setattr__(self, "mixer_norm", norms.get("mixer"))
        object.__setattr__(self, "feed_forward_norm", norms.get("feed_forward"))


@dataclass(frozen=True)
class RunEntry:
    """One position of the run order.  `block` indexes `ModelSpec.blocks` and may appear
    in several entries.  `cache` is the cache entry the mixer uses; entries that name the
    same `cache` share keys and values, and only the entry with `writes_cache` stores
    into it (the other reads what the first one wrote in the same step)."""
    block: int
    cache: int
    writes_cache: bool = True


@dataclass(frozen=True)
class ModelSpec:
    """`embedding` and `head` are parts like the others; a model with the plain table at both
    ends gives their tensor names instead (`embedding_name`, and `head_name`, None for a head
    tied to the table) and gets the built-in `token_embedding` and `linear_head`."""
    hidden_size: int
    vocab_size: int
    final_norm: PartSpec
    blocks: Tuple[BlockSpec, ...]
    schedule: Tuple[RunEntry, ...]
    max_positions: int
    embedding_name: Optional[str] = None
    head_name: Optional[str] = None   # None: the head is the embedding table (tied)
    stop_tokens: Tuple[int, ...] = ()
    embedding: Optional[PartSpec] = None
    head: Optional[PartSpec] = None

    def __post_init__(self):
        sizes = dict(vocab_size=self.vocab_size, hidden_size=self.hidden_size)
        if self.embedding is None:
            if self.embedding_name is None:
                raise ValueError("ModelSpec needs an embedding part or the embedding table's tensor name")
            object.__setattr__(self, "embedding", PartSpec("token_embedding", dict(sizes, name=self.embedding_name)))
        if self.head is None:
            object.__setattr__(self, "head", PartSpec("linear_head", dict(sizes, name=self.head_name)))
        for e in self.schedule:
            if not 0 <= e.block < len(self.blocks):
                raise ValueError(f"schedule names block {e.block}, model has {len(self.blocks)}")
        writers = {}
        for n, e in enumerate(self.schedule):
            if e.writes_cache:
                if e.cache in writers:
                    raise ValueError(f"cache entry {e.cache} is written by schedule positions "
                                     f"{writers[e.cache]} and {n}")
                writers[e.cache] = n
        for n, e in enumerate(self.schedule):
            if not e.writes_cache and (e.cache not in writers or writers[e.cache] > n):
                raise ValueError(f"schedule position {n} reads cache entry {e.cache} "
                                 "before any position writes it")


def straight_schedule(n_blocks: int) -> Tuple[RunEntry, ...]:
    """Block i runs i-th and owns cache entry i."""
    return tuple(RunEntry(block=i, cache=i) for i in range(n_blocks))

"""A decoder model put together from a `ModelSpec`: embedding, blocks in their run order,
final norm, head.  Which parts, with which constants, comes from the spec alone.

One step (src/models/qwen2/graph.rs:36-185 of yusiwen/minfer): rows of the embedding table
-> every entry of the run order -> only the wanted rows go through the last block's
feed-forward, the final norm and the head (the reference's tail-row reduction,
graph.rs:126-138) -> float32 logits.
"""
from __future__ import annotations

from typing import Callable, Dict

import torch

from ..kernels import ops, tuning
from ..parts.base import (BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, Runtime, make_part,
                          normed_input)
from ..parts.spec import BlockSpec, ModelSpec
from ..weights.loader import TensorSpec


def _build_block(bs: BlockSpec, rt: Runtime):
    """The block's arrangement and the parts its spec names; the arrangement says which it needs."""
    if bs.kind not in BLOCKS:
        raise KeyError(f"unknown block arrangement {bs.kind!r}; registered: {', '.join(sorted(BLOCKS))}")
    cls = BLOCKS[bs.kind]
    where = f"block {bs.prefix!r} ({bs.kind})"
    if cls.needs_mixer and bs.mixer is None:
        raise ValueError(f"{where}: this arrangement needs a mixer")
    if cls.needs_feed_forward and bs.feed_forward is None:
        raise ValueError(f"{where}: this arrangement needs a feed-forward")
    known = tuple(cls.norm_names) + tuple(cls.optional_norms)
    missing = [n for n in cls.norm_names if n not in bs.norms]
    unknown = [n for n in bs.norms if n not in known]
    if missing or unknown:
        raise ValueError(f"{where}: norms missing {missing}, not known to the arrangement {unknown}; "
                         f"it takes {list(known)}")
    return cls(None if bs.mixer is None else make_part(MIXERS, bs.mixer, rt, "mixer"),
               None if bs.feed_forward is None else make_part(FEED_FORWARDS, bs.feed_forward, rt, "feed-forward"),
               {name: make_part(NORMS, spec, rt, "norm") for name, spec in bs.norms.items()}, rt)


class DecoderModel:
    def __init__(self, spec: ModelSpec, dtype: torch.dtype, device):
        if dtype not in (torch.float32, torch.bfloat16):
            raise ValueError(f"run type must be float32 or bfloat16, got {dtype}")
        self.spec = spec
        self.rt = Runtime(dtype=dtype, device=torch.device(device))
        self.blocks = [_build_block(bs, self.rt) for bs in spec.blocks]
        self.final_norm = make_part(NORMS, spec.final_norm, self.rt, "norm")
        self.embedding = make_part(EMBEDDINGS, spec.embedding, self.rt, "embedding")
        self.head = make_part(HEADS, spec.head, self.rt, "head")
        self.stop_tokens = tuple(spec.stop_tokens)      # a loader may add to them (generation_config.json)
        self.loaded = False
        self.decode_copy_bytes = 0      # of the parts' tiled second copies, once loaded

    # ------------------------------------------------------------ tensors
    def expected_tensors(self) -> Dict[str, TensorSpec]:
        s = self.spec
        out: Dict[str, TensorSpec] = {}
        for part in (self.embedding, self.head, self.final_norm):
            for name, ts in part.tensor_specs().items():
                if name in out:
                    raise ValueError(f"tensor {name!r} is claimed by two parts")
                out[name] = ts
        for bs, block in zip(s.blocks, self.blocks):
            for part in block.parts():
                for name, ts in part.tensor_specs().items():
                    full = bs.prefix + name
                    if full in out:
                        raise ValueError(f"tensor {full!r} is claimed by two parts")
                    out[full] = ts
        return out

    def load(self, get: Callable[[str], torch.Tensor]) -> None:
        """`get(full name)` returns a device tensor in its storage type."""
        s = self.spec
        self.embedding.load(get)
        self.head.load(get)
        self.head.tie(self.embedding)        # a tied head takes the table's storage, no second copy
        self.final_norm.load(get)
        for bs, block in zip(s.blocks, self.blocks):
            for part in block.parts():
                part.load(lambda name, p=bs.prefix: get(p + name))
        self.loaded = True
        self.decode_copy_bytes = self._make_decode_copies()

    def _all_parts(self):
        yield from (self.embedding, self.head, self.final_norm)
        for block in self.blocks:
            yield from block.parts()

    def _make_decode_copies(self) -> int:
        """The parts' second copies of their matrices for the steps of few tokens (a layout that
        those steps' products read faster): of all matrices where that takes at most a third of
        the device memory that is free once the weights are in place, else of those with rows of
        16,384 and more (the down products, which gain most) under the same condition, else
        none, so that a model that fills the device keeps its memory for the cache.  Returns
        their bytes."""
        if not self.rt.is_bf16 or self.rt.device.type != "cuda" or tuning.NO_DECODE_COPIES:
            return 0
        free, _ = torch.cuda.mem_get_info(self.rt.device)
        for min_row_length in (0, 16384):
            need = sum(part.decode_copies(False, min_row_length) for part in self._all_parts())
            if 0 < need <= free // 3:
                return sum(part.decode_copies(True, min_row_length) for part in self._all_parts())
        return 0

    # ------------------------------------------------------------ cache needs
    def cache_requests(self) -> Dict[int, object]:
        """cache entry -> what the mixer that writes it asks for."""
        return {e.cache: None if self.blocks[e.block].mixer is None else self.blocks[e.block].mixer.cache_request()
                for e in self.spec.schedule if e.writes_cache}

    def prepare(self, max_len: int) -> None:
        for part in (self.embedding, self.head, self.final_norm):
            part.prepare(max_len)
        for block in self.blocks:
            for part in block.parts():
                part.prepare(max_len)

    # ------------------------------------------------------------ the step
    def forward(self, ctx) -> torch.Tensor:
        """float32 logits [n_wanted][vocab] for ctx.logit_rows (all rows when None)."""
        if not self.loaded:
            raise RuntimeError("model has no weights yet")
        s = self.spec
        h = torch.empty((ctx.n_tokens, s.hidden_size), dtype=torch.float32, device=self.rt.device)
        self.embedding.forward(ctx.token_ids, h, ctx)
        rows = ctx.logit_rows
        last = len(s.schedule) - 1
        ctx.norm_ahead = None
        for n, e in enumerate(s.schedule):
            keep = rows if (n == last and rows is not None) else None
            # the norm that reads the stream behind this block: the next block's first one, or the final one
            ctx.norm_after_block = (self.final_norm if n == last else self.blocks[s.schedule[n + 1].block].first_norm())
            h = self.blocks[e.block].forward(h, ctx, e.cache, e.writes_cache, keep_rows=keep)
            ahead = ctx.norm_ahead
            if ahead is not None and (ahead.norm is not ctx.norm_after_block or ahead.h is not h):
                ctx.norm_ahead = None            # prepared for someone who will not come
        ctx.norm_after_block = None
        if not s.schedule and rows is not None:
            kept = torch.empty((rows.numel(), s.hidden_size), dtype=torch.float32, device=h.device)
            ops.gather_rows(h, rows, kept)
            h = kept
        return self.head.forward(normed_input(self.final_norm, self.head, h, ctx=ctx), ctx)


def expected_tensors(spec: ModelSpec) -> Dict[str, TensorSpec]:
    """Names, shapes and fill rules of a spec's tensors, without touching a device."""
    return DecoderModel(spec, torch.float32, "cpu").expected_tensors()

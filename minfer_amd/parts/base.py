"""Interfaces of the parts a block is put together from, and the registries that map a
`PartSpec.kind` to a class.

A part is built from its constants alone (`PartSpec.params`), says which tensors it wants
(`tensor_specs`, names relative to the block's prefix), receives them (`load`), and runs.
It never sees the configuration, the model, or which layer it is.  The step's ragged batch
arrives as a `StepContext` (see `minfer_amd.engine.batch`).

Numeric contract between parts: the residual stream `h` is float32 `[tokens][hidden]`;
norms read it and write the run type (bfloat16 or float32); mixers and feed-forwards read
the run type and *add* their result into `h` in 32-bit.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Dict, Optional

import torch

from ..weights.loader import TensorSpec
from .spec import PartSpec


@dataclass
class Runtime:
    """Where and in which precision a model runs."""
    dtype: torch.dtype          # run type of activations, matrices and cache
    device: torch.device

    @property
    def is_bf16(self) -> bool:
        return self.dtype == torch.bfloat16


class Part:
    """Base of every part."""

    def __init__(self, spec: PartSpec, rt: Runtime):
        self.spec, self.rt = spec, rt

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {}

    def load(self, get: Callable[[str], torch.Tensor]) -> None:
        """`get(name)` returns the tensor on the device in its storage type."""

    def prepare(self, max_len: int) -> None:
        """Called before steps that may reach `max_len` positions (tables, workspaces), so
        that a captured step allocates nothing of its own."""

    def decode_copies(self, make: bool, min_row_length: int = 0) -> int:
        """Bytes of the second copies of its matrices (those with rows of at least
        `min_row_length`) that this part would keep for the steps of few tokens
        (`Linear.decode_copy`); made when `make`.  The model asks all parts first and makes the
        copies only where the device has the memory to spare."""
        return 0


class Norm(Part):
    def forward(self, h: torch.Tensor, out: Optional[torch.Tensor] = None,
                row_idx: Optional[torch.Tensor] = None) -> torch.Tensor:
        """float32 rows in, run-type rows out; row r reads h[row_idx[r]] when given."""
        raise NotImplementedError

    def rms_scale(self):
        """(weight, eps) if this norm is y = x / sqrt(mean(x^2) + eps) * weight with a float32
        weight vector, else None.  A product that follows such a norm may fold it in."""
        return None


@dataclass
class NormAhead:
    """What a product that added into the residual stream `h` left for `norm`, the norm that reads
    the stream next: bf16(h g) and, per row, partial sums of h^2 (`ops.linear_fused`).  The product
    that follows the norm may take these instead of the normed rows."""
    norm: "Norm"
    h: torch.Tensor
    xg: torch.Tensor
    sums: torch.Tensor


class Normed:
    """The rows `norm(h[row_idx])` before anyone has computed them.  A block hands this to a
    mixer or feed-forward that declares `takes_normed = True`; such a part passes it to its
    first `Linear`, which folds the norm into the product where a kernel for that exists, or
    calls `tensor()` (computed once, then kept) like any part that needs the rows themselves.
    `ahead`: what the product before the norm prepared for it, if it did."""

    def __init__(self, norm: "Norm", h: torch.Tensor, row_idx: Optional[torch.Tensor] = None,
                 ahead: Optional[NormAhead] = None):
        self.norm, self.h, self.row_idx = norm, h, row_idx
        self.ahead = ahead
        self._rows: Optional[torch.Tensor] = None

    @property
    def shape(self):
        return (self.h.shape[0] if self.row_idx is None else self.row_idx.numel(), self.h.shape[1])

    @property
    def device(self):
        return self.h.device

    def tensor(self) -> torch.Tensor:
        if self._rows is None:
            self._rows = self.norm.forward(self.h, row_idx=self.row_idx)
        return self._rows


def normed_input(norm: "Norm", part, h: torch.Tensor, row_idx: Optional[torch.Tensor] = None, ctx=None):
    """What a block gives `part` as its input: the lazy form if the part takes it.  With `ctx`,
    whatever the product before left for this norm over these rows (`ctx.norm_ahead`) goes along,
    and is taken off the context either way: it describes the stream as it is now."""
    ahead = None
    if ctx is not None:
        ahead, ctx.norm_ahead = getattr(ctx, "norm_ahead", None), None
        if ahead is not None and (ahead.norm is not norm or ahead.h is not h or row_idx is not None):
            ahead = None
    if getattr(part, "takes_normed", False):
        return Normed(norm, h, row_idx, ahead)
    return norm.forward(h, row_idx=row_idx)


def announce_norm(ctx, norm: Optional["Norm"]) -> None:
    """A block says which norm reads the residual stream after the part it is about to run (None:
    nobody it knows of).  A part whose last product adds into the stream may pass `ctx` on to it
    (`Linear(..., ctx=ctx)`), and the product may then prepare that norm's input (`NormAhead`)."""
    ctx.norm_next = norm
    ctx.norm_ahead = None


class PositionEncoding(Part):
    """Puts the tokens' positions into queries and keys.  Storing keys and values is not its
    business: the cache does that (`Cache.store_kv`), so an encoding knows nothing of pages."""

    def encode(self, qkv: torch.Tensor, ctx, n_heads: int, n_kv_heads: int) -> None:
        """Encodes `ctx.positions` into the q heads (the first `n_heads`) and the k heads (the next
        `n_kv_heads`) of the 32-bit `[tokens][(n_heads + 2 n_kv_heads) head_dim]` rows, in place;
        the v heads stay as they are."""
        raise NotImplementedError

    def rotation_tables(self, max_len: int):
        """(cos, sin) `[positions][head_dim / 2]` float32 tables if this encoding is the half-split
        rotation, else None.  A mixer may then use kernels that rotate on the way (rotation and
        cache write in one, or inside the decode attention) instead of calling `encode`."""
        return None


class Mixer(Part):
    def cache_request(self):
        """A `KVRequest`, a `StateRequest` or None."""
        return None

    takes_normed = False     # True: `x` may arrive as a `Normed` (see there)

    def forward(self, x: torch.Tensor, h: torch.Tensor, ctx, entry: int, writes_cache: bool) -> None:
        """Adds the mixer's output for the step's tokens into h.  `entry` is the cache entry
        (`ctx.cache.kv(entry)` / `ctx.cache.state(entry)`)."""
        raise NotImplementedError


class FeedForward(Part):
    takes_normed = False     # True: `x` may arrive as a `Normed`

    def forward(self, x: torch.Tensor, h: torch.Tensor, ctx) -> None:
        """Adds the feed-forward's output into h (h may hold fewer rows than the step)."""
        raise NotImplementedError


class Embedding(Part):
    """Token ids in, rows of the 32-bit residual stream out."""

    def forward(self, token_ids: torch.Tensor, out: torch.Tensor, ctx) -> None:
        """Writes the row of every id (int32 on the device) into `out` (float32 `[tokens][hidden]`).
        `ctx` is the step (positions, sequences), for an embedding that depends on where a token
        stands."""
        raise NotImplementedError

    def table(self) -> Optional[torch.Tensor]:
        """The `[vocab][hidden]` matrix a tied head multiplies by, if this embedding has one."""
        return None


class Head(Part):
    """The wanted rows of the residual stream, after the final norm, to float32 logits."""

    def tie(self, embedding: "Embedding") -> None:
        """Called once after loading when the head shares the embedding's storage."""

    def forward(self, x, ctx) -> torch.Tensor:
        """`x`: the final norm's rows, as a tensor or (when `takes_normed`) a `Normed`: the step's
        rows `ctx.logit_rows` (all of them when that is None), in that order.  Returns float32
        `[rows][vocab]`."""
        raise NotImplementedError

    takes_normed = False


class Block:
    """An arrangement of parts: a mixer and a feed-forward (either may be None where the
    arrangement allows it) and norms under the names the arrangement gives them (`norm_names`;
    `optional_norms` may be left out).  `forward` returns the residual stream, reduced to the rows
    `keep_rows` (int32 indices on the device) when given."""

    norm_names = ("mixer", "feed_forward")
    optional_norms = ()
    needs_mixer = True
    needs_feed_forward = True

    def __init__(self, mixer: Optional[Mixer], feed_forward: Optional[FeedForward], norms: Dict[str, Norm],
                 rt: Runtime):
        self.mixer, self.feed_forward = mixer, feed_forward
        self.norms = dict(norms)
        self.rt = rt

    @property
    def mixer_norm(self) -> Optional[Norm]:
        return self.norms.get("mixer")

    @property
    def feed_forward_norm(self) -> Optional[Norm]:
        return self.norms.get("feed_forward")

    def parts(self):
        """Every part of the block that exists, norms in the order of `norm_names`."""
        named = [self.norms[n] for n in self.norm_names + self.optional_norms if n in self.norms]
        return tuple(p for p in [self.mixer, self.feed_forward] + named if p is not None)

    def first_norm(self) -> Optional[Norm]:
        """The norm that reads the residual stream first when this block runs, if it starts with
        one (the block before may then prepare its input, see `announce_norm`)."""
        return None

    def forward(self, h, ctx, entry: int, writes_cache: bool, keep_rows=None):
        raise NotImplementedError


MIXERS: Dict[str, type] = {}
FEED_FORWARDS: Dict[str, type] = {}
NORMS: Dict[str, type] = {}
POSITIONS: Dict[str, type] = {}
BLOCKS: Dict[str, type] = {}
EMBEDDINGS: Dict[str, type] = {}
HEADS: Dict[str, type] = {}


def _registrar(table: Dict[str, type], what: str):
    def register(kind: str):
        def deco(cls):
            table[kind] = cls
            return cls
        return deco
    register.__doc__ = f"Class decorator: registers a {what} under a PartSpec.kind."
    return register


register_mixer = _registrar(MIXERS, "mixer")
register_feed_forward = _registrar(FEED_FORWARDS, "feed-forward")
register_norm = _registrar(NORMS, "norm")
register_position = _registrar(POSITIONS, "position encoding")
register_block = _registrar(BLOCKS, "block arrangement")
register_embedding = _registrar(EMBEDDINGS, "embedding")
register_head = _registrar(HEADS, "head")


def make_part(table: Dict[str, type], spec: PartSpec, rt: Runtime, what: str):
    if spec.kind not in table:
        raise KeyError(f"unknown {what} {spec.kind!r}; registered: {', '.join(sorted(table)) or '(none)'}")
    return table[spec.kind](spec, rt)

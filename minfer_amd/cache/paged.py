"""The cache: a slot per live sequence, keys and values per cache entry in pages of 64
tokens, and a fixed-size state area per slot.

The reference keeps, per layer, two regions `[n_ctx][n_kv]` whose row index is the absolute
position, never zeroes them, and reads rows `0..=pos` only, so a reused cache needs no
clearing (src/graph/alloc.rs:258-279, src/graph/cpu_backend.rs:139-147,462 of
yusiwen/minfer); a server slot owns one such cache and goes Idle -> Processing -> Idle
(src/server/slot.rs:7-32).  Here the rows of a sequence live in pages drawn from a pool, so
the pool is sized in tokens (each sequence rounded up to whole pages), not in slots x
context.  The same rule makes reuse safe: a page's old rows are never read, because a
sequence reads positions below its own length only and writes each before reading it.

Layers with the same needs (kv heads, head size, window, value width) form a group with storage
of its own: one K tensor `[entries][pages][kv_heads][64][head_dim]`, one V tensor (the same shape
in 32-bit, `[entries][pages][kv_heads][2][head_dim][32]` in bfloat16, see `v_page_shape`; with the
request's own value width where it names one) and one page pool.
A group with a window gives pages back as soon as every position in them has left the
window of all later queries.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import torch

PAGE = 64


V_HALF = PAGE // 2


def v_page_shape(n_kv_heads: int, head_dim: int, dtype) -> Tuple[int, ...]:
    """One page of V: like K, `[kv_heads][64][head_dim]`, in 32-bit.  In bfloat16 it is transposed
    in two halves of 32 keys, `[kv_heads][2][head_dim][32]` (key j of the page is element j % 32
    of half j / 32): the attention kernels feed V^T rows to the matrix cores as they are stored,
    32 keys at a time, and what 16 lanes-rows of such a step read is one contiguous kilobyte."""
    if dtype == torch.bfloat16:
        return (n_kv_heads, 2, head_dim, V_HALF)
    return (n_kv_heads, PAGE, head_dim)


class CacheError(RuntimeError):
    pass


class CacheFull(CacheError):
    """Not enough free pages or slots; nothing was changed."""


@dataclass(frozen=True)
class KVRequest:
    """What an attention-like mixer asks of the cache for one entry."""
    n_kv_heads: int
    head_dim: int
    window: Optional[int] = None      # None: all earlier positions
    v_head_dim: Optional[int] = None  # width of a value row where it is not that of a key row

    @property
    def value_dim(self) -> int:
        return self.head_dim if self.v_head_dim is None else self.v_head_dim


@dataclass(frozen=True)
class StateRequest:
    """Fixed-size state per sequence for one entry (zeroed when a slot is taken)."""
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


class PagePool:
    """Free list of page ids with double-free and leak checks (host side only)."""

    def __init__(self, n_pages: int):
        self.n_pages = n_pages
        self._free = list(range(n_pages - 1, -1, -1))
        self._held = [False] * n_pages

    @property
    def free_pages(self) -> int:
        return len(self._free)

    def take(self, n: int) -> List[int]:
        if n > len(self._free):
            raise CacheFull(f"cache needs {n} more pages of {PAGE} tokens, {len(self._free)} of "
                            f"{self.n_pages} are free")
        pages = [self._free.pop() for _ in range(n)]
        for p in pages:
            self._held[p] = True
        return pages

    def give(self, pages: Sequence[int]) -> None:
        for p in pages:
            if not 0 <= p < self.n_pages or not self._held[p]:
                raise CacheError(f"page {p} given back but not held")
            self._held[p] = False
            self._free.append(p)


class KVGroup:
    """Storage and page bookkeeping of the entries that share one KVRequest."""

    def __init__(self, request: KVRequest, entries: List[int], n_pages: int, dtype, device,
                 poison: bool = False):
        self.poison = poison
        self.request = request
        self.entries = list(entries)
        self.index_of = {e: i for i, e in enumerate(self.entries)}
        self.pool = PagePool(n_pages)
        self.k = torch.empty((len(entries), n_pages, request.n_kv_heads, PAGE, request.head_dim),
                             dtype=dtype, device=device)
        self.v = torch.empty((len(entries), n_pages) + v_page_shape(request.n_kv_heads, request.value_dim, dtype),
                             dtype=dtype, device=device)
        if poison:
            self.k.fill_(float("nan"))
            self.v.fill_(float("nan"))
        self.pages: Dict[int, List[int]] = {}      # slot -> page id per logical page, -1 = given back

    def _give(self, pages: List[int]) -> None:
        """Back to the pool.  With `poison` (tests) the pages are overwritten with NaN, so that
        a read of a row its sequence never wrote shows at once."""
        self.pool.give(pages)
        if self.poison and pages:
            idx = torch.tensor(pages, dtype=torch.long, device=self.k.device)
            self.k[:, idx] = float("nan")
            self.v[:, idx] = float("nan")

    def first_needed_page(self, length: int) -> int:
        """Lowest logical page a query at position >= length can still read."""
        w = self.request.window
        if w is None:
            return 0
        return max(0, length - w + 1) // PAGE

    def pages_missing(self, slot: int, new_len: int) -> int:
        return max(0, (new_len + PAGE - 1) // PAGE - len(self.pages[slot]))

    def grow(self, slot: int, new_len: int) -> None:
        self.pages[slot].extend(self.pool.take(self.pages_missing(slot, new_len)))

    def shrink_to(self, slot: int, length: int) -> None:
        """Gives back pages above `length` (truncate) ."""
        keep = (length + PAGE - 1) // PAGE
        tail = [p for p in self.pages[slot][keep:] if p >= 0]
        del self.pages[slot][keep:]
        self._give(tail)

    def drop_left_of_window(self, slot: int, length: int) -> None:
        first = self.first_needed_page(length)
        row = self.pages[slot]
        gone = [p for p in row[:first] if p >= 0]
        for i in range(min(first, len(row))):
            row[i] = -1
        self._give(gone)

    def release(self, slot: int) -> None:
        self._give([p for p in self.pages.pop(slot) if p >= 0])


class Cache:
    """`requests[entry]` is a KVRequest, a StateRequest or None, one per cache entry of the
    model's run order.  `max_tokens` is the most tokens all live sequences hold together,
    each rounded up to a multiple of 64; `max_seqs` bounds the live sequences.  `poison`
    (tests) fills pages with NaN when they are created and whenever they are given back."""

    def __init__(self, requests: Dict[int, object], max_tokens: int, max_seqs: int, dtype, device,
                 poison: bool = False):
        if max_tokens < 1 or max_seqs < 1:
            raise CacheError("cache needs room for at least one token and one sequence")
        self.dtype, self.device = dtype, device
        self.n_pages = (max_tokens + PAGE - 1) // PAGE
        self.max_seqs = max_seqs
        by_request: Dict[KVRequest, List[int]] = {}
        self.state_requests: Dict[int, StateRequest] = {}
        for entry, req in sorted(requests.items()):
            if isinstance(req, KVRequest):
                by_request.setdefault(req, []).append(entry)
            elif isinstance(req, StateRequest):
                self.state_requests[entry] = req
            elif req is not None:
                raise CacheError(f"cache entry {entry}: unknown request {req!r}")
        self.groups: List[KVGroup] = [KVGroup(r, es, self.n_pages, dtype, device, poison)
                                      for r, es in by_request.items()]
        self.group_of: Dict[int, KVGroup] = {e: g for g in self.groups for e in g.entries}
        self.states: Dict[int, torch.Tensor] = {
            e: torch.zeros((max_seqs,) + tuple(r.shape), dtype=r.dtype, device=device)
            for e, r in self.state_requests.items()}
        self._free_slots = list(range(max_seqs - 1, -1, -1))
        self.lengths: Dict[int, int] = {}          # live slot -> tokens held

    # ------------------------------------------------------------ slots
    def alloc_slot(self) -> int:
        if not self._free_slots:
            raise CacheFull(f"all {self.max_seqs} sequence slots are in use")
        slot = self._free_slots.pop()
        self.lengths[slot] = 0
        for g in self.groups:
            g.pages[slot] = []
        for s in self.states.values():
            s[slot].zero_()
        return slot

    def free_slot(self, slot: int) -> None:
        if slot not in self.lengths:
            raise CacheError(f"slot {slot} freed but not in use")
        for g in self.groups:
            g.release(slot)
        del self.lengths[slot]
        self._free_slots.append(slot)

    def live_slots(self) -> List[int]:
        return sorted(self.lengths)

    def length(self, slot: int) -> int:
        if slot not in self.lengths:
            raise CacheError(f"slot {slot} is not in use")
        return self.lengths[slot]

    # ------------------------------------------------------------ growth
    def reserve(self, new_lengths: Dict[int, int]) -> None:
        """Pages for every position below new_lengths[slot] in every group, for all the
        given slots or for none (CacheFull)."""
        for slot, n in new_lengths.items():
            if n < self.length(slot):
                raise CacheError(f"slot {slot}: reserve({n}) below its length {self.lengths[slot]}")
        for g in self.groups:
            need = sum(g.pages_missing(s, n) for s, n in new_lengths.items())
            if need > g.pool.free_pages:
                raise CacheFull(f"cache needs {need} more pages of {PAGE} tokens, "
                                f"{g.pool.free_pages} of {g.pool.n_pages} are free")
        for g in self.groups:
            for s, n in new_lengths.items():
                g.grow(s, n)

    def commit(self, new_lengths: Dict[int, int]) -> None:
        """The step wrote positions up to new_lengths[slot]: record it, and let windowed
        groups give back pages no later query can read."""
        for slot, n in new_lengths.items():
            self.lengths[slot] = n
            for g in self.groups:
                if g.request.window is not None:
                    g.drop_left_of_window(slot, n)

    def truncate(self, slot: int, length: int) -> None:
        """Rolls a sequence back; rows above are simply never read again
        (src/conversation.rs:334-349).  Not possible once a window has dropped pages that
        the shorter sequence would need, or for entries with fixed-size state."""
        if length > self.length(slot) or length < 0:
            raise CacheError(f"slot {slot}: truncate({length}) outside [0, {self.lengths[slot]}]")
        if self.states and length != self.lengths[slot]:
            raise CacheError("truncate: this model keeps per-sequence state that cannot be rolled back")
        for g in self.groups:
            first = g.first_needed_page(length)
            if any(p < 0 for p in g.pages[slot][first:(length + PAGE - 1) // PAGE]):
                raise CacheError("truncate: a windowed group already gave back pages this length needs")
        for g in self.groups:
            g.shrink_to(slot, length)
        self.lengths[slot] = length

    # ------------------------------------------------------------ views
    def kv(self, entry: int):
        """(K, V) of one entry, `[pages]` + page shape each, and its group."""
        g = self.group_of[entry]
        i = g.index_of[entry]
        return g.k[i], g.v[i], g

    def store_kv(self, entry: int, qkv: torch.Tensor, ctx, n_heads: int, q_out: torch.Tensor) -> None:
        """Stores the step's keys and values into the entry's pages at the tokens' positions and
        leaves q, rounded to the run type, in `q_out`.  `qkv` is the 32-bit
        `[tokens][(n_heads + 2 kv_heads) head_dim]` row of q|k|v with every position encoding
        already applied.  The page layout (`v_page_shape`) is known here and in the kernels only:
        a mixer or a position encoding never indexes pages itself."""
        from ..kernels import ops
        k, v, group = self.kv(entry)
        req = group.request
        if req.value_dim != req.head_dim:
            raise CacheError(f"store_kv writes keys and values of one width; entry {entry} asks for keys of "
                             f"{req.head_dim} and values of {req.value_dim}: a mixer with a value width of its own "
                             "writes its rows into the pages of `kv(entry)` with a kernel of its own")
        ops.rope_kvwrite(qkv, None, None, ctx.positions, ctx.seq_of_tok, ctx.page_table(group), q_out, k, v,
                         n_heads, req.n_kv_heads, req.head_dim, True)

    def state(self, entry: int) -> torch.Tensor:
        """The entry's fixed-size state of every slot, `[max_seqs] + shape`.  A step addresses its
        sequences' rows with `ctx.slot_ids` (int32 on the device), e.g.
        `state.index_select(0, ctx.slot_ids.long())` and `state.index_copy_`: the slots are data,
        so a captured decode step serves whichever slots it is bound to."""
        return self.states[entry]

    def page_rows(self, group: KVGroup, slots: Sequence[int], n_cols: int) -> List[List[int]]:
        """Page table rows of `slots`, padded with -1 to n_cols."""
        rows = []
        for s in slots:
            row = group.pages[s]
            if len(row) > n_cols:
                raise CacheError(f"slot {s} holds {len(row)} pages, table has {n_cols} columns")
            rows.append(row + [-1] * (n_cols - len(row)))
        return rows

    def free_tokens(self) -> int:
        return min((g.pool.free_pages for g in self.groups), default=self.n_pages) * PAGE

    def check_invariants(self) -> None:
        """No page lost, held twice or free twice; used by tests."""
        for g in self.groups:
            held = [p for row in g.pages.values() for p in row if p >= 0]
            if len(held) != len(set(held)):
                raise CacheError("a page is held by two sequences")
            free = g.pool._free
            if len(free) != len(set(free)) or set(free) & set(held):
                raise CacheError("a page is free twice, or free and held")
            if len(free) + len(held) != g.pool.n_pages:
                raise CacheError(f"{g.pool.n_pages - len(free) - len(held)} pages lost")
            if set(g.pages) != set(self.lengths):
                raise CacheError("page rows and live slots disagree")
        if len(set(self._free_slots)) != len(self._free_slots) or \
                set(self._free_slots) & set(self.lengths) or \
                len(self._free_slots) + len(self.lengths) != self.max_seqs:
            raise CacheError("slot lost, held twice or freed twice")

"""The step function: a batch of sequences with unequal numbers of new tokens, run as one
ragged batch from the cache, logits returned at the wanted places.

The reference's step is `forward(tokens, positions, n_out) -> n_out x vocab logits` for one
sequence per call, with a prompt as one call and then one token per call
(src/models/mod.rs:21-22, src/models/qwen2/graph.rs:276-408, src/main.rs:497-502,595 of
yusiwen/minfer); a batch there is one call per cache (src/server/chat.rs:218-249).  Here the
whole batch is one call: tokens of all sequences concatenated, per-token position and
sequence index as data.  There is no padding: only the tokens given are run.
"""
from __future__ import annotations

from collections import OrderedDict
from typing import Dict, Optional, Sequence, Union

import numpy as np
import torch

from ..cache.paged import PAGE, Cache, CacheError
from .batch import StepContext
from .model import DecoderModel

Want = Union[str, Sequence[Sequence[int]]]


class StepError(ValueError):
    """A step that cannot run: the message says which sequence and why.  Nothing changed."""


# Decode sessions an engine keeps (each holds a captured graph with a memory pool of its own: the
# logits of its batch size and the activations of a step); the least recently used one goes first.
MAX_SESSIONS = 8

# Device memory left alone when the cache is sized from what is free: the activations and logits
# of the largest step, workspaces of the kernels, the pools of captured graphs.
RESERVE_BYTES_MIN = 2 << 30
RESERVE_FRACTION = 0.06


def cache_bytes_per_token(requests: Dict[int, object], dtype: torch.dtype) -> int:
    """Bytes one token of one sequence takes in the cache: K and V of every entry."""
    from ..cache.paged import KVRequest
    elem = torch.empty((), dtype=dtype).element_size()
    return sum(r.n_kv_heads * (r.head_dim + r.value_dim) * elem for r in requests.values() if isinstance(r, KVRequest))


def state_bytes_per_sequence(requests: Dict[int, object]) -> int:
    """Bytes of fixed-size state one sequence slot takes, over all entries that ask for state."""
    from ..cache.paged import StateRequest
    total = 0
    for r in requests.values():
        if isinstance(r, StateRequest):
            n = torch.empty((), dtype=r.dtype).element_size()
            for d in r.shape:
                n *= int(d)
            total += n
    return total


# Sequence slots assumed for the fixed-size state when the caller names no number of sequences
DEFAULT_STATE_SLOTS = 1024


def plan_cache_tokens(free: int, total: int, per_token: int, state_bytes: int, step_bytes: int) -> int:
    """Tokens (whole pages) a cache can hold in `free` bytes of a device of `total` bytes, after
    the reserve (the larger of RESERVE_BYTES_MIN and RESERVE_FRACTION of the device), the
    activations of the largest step (`step_bytes`) and the sequences' fixed-size state
    (`state_bytes`, for all slots).  CacheError where not even one page fits."""
    reserve = max(RESERVE_BYTES_MIN, int(RESERVE_FRACTION * total)) + int(step_bytes) + int(state_bytes)
    per_token = max(1, int(per_token))
    tokens = (int(free) - reserve) // per_token // PAGE * PAGE
    if tokens < PAGE:
        raise CacheError(f"no room for a cache: {int(free) >> 20} MiB free, {reserve >> 20} MiB held back "
                         f"({int(state_bytes) >> 20} MiB of them per-sequence state), {per_token} bytes a token")
    return int(tokens)


def tokens_that_fit(model: DecoderModel, max_step_tokens: int = 8192, max_seqs: Optional[int] = None,
                    mem_info=None) -> int:
    """How many tokens the cache can hold in the device memory that is free now (the weights are
    loaded), after a reserve for everything else a step needs and the fixed-size state of
    `max_seqs` sequences.  The reference divides a given context over its slots
    (src/server/slot.rs:27-32 of yusiwen/minfer); here the given is what the GPU has left.
    `mem_info()` returns (free, total) bytes; by default the device's own figures."""
    if mem_info is None:
        if model.rt.device.type != "cuda":
            return 1 << 30                   # (tests drive the engine through stand-ins on the host)
        mem_info = lambda: torch.cuda.mem_get_info(model.rt.device)
    free, total = mem_info()
    requests = model.cache_requests()
    step = max_step_tokens * model.spec.hidden_size * 4 * 12      # residual, q|k|v, feed-forward rows of a large step
    state = state_bytes_per_sequence(requests) * int(max_seqs or DEFAULT_STATE_SLOTS)
    return plan_cache_tokens(free, total, cache_bytes_per_token(requests, model.rt.dtype), state, step)


class Engine:
    def __init__(self, model: DecoderModel, max_tokens: Optional[int] = None, max_seqs: Optional[int] = None,
                 poison_cache: bool = False):
        """`max_tokens`: the most tokens all live sequences hold together (each rounded up to whole
        pages of 64); None: as many as fit into the device memory that is free after the weights
        (`tokens_that_fit`)."""
        if not model.loaded:
            raise RuntimeError("Engine needs a model with weights")
        self.model = model
        self.device = model.rt.device
        if max_tokens is None:
            max_tokens = tokens_that_fit(model, max_seqs=max_seqs)
            if max_seqs:
                max_tokens = min(max_tokens, int(max_seqs) * ((model.spec.max_positions + PAGE - 1) // PAGE * PAGE))
        n_pages = (max_tokens + PAGE - 1) // PAGE
        self.max_seqs = int(max_seqs) if max_seqs else max(1, min(n_pages, 1024))
        self.cache = Cache(model.cache_requests(), max_tokens, self.max_seqs, model.rt.dtype, self.device,
                           poison=poison_cache)
        self.vocab_size = model.spec.vocab_size
        self.max_positions = model.spec.max_positions
        self._sessions: "OrderedDict" = OrderedDict()

    # ------------------------------------------------------------ sequences
    def new_sequence(self) -> int:
        """Takes a cache slot for a sequence that starts at position 0."""
        return self.cache.alloc_slot()

    def end_sequence(self, slot: int) -> None:
        """Gives the slot and everything it holds back."""
        self.cache.free_slot(slot)

    def length(self, slot: int) -> int:
        return self.cache.length(slot)

    def capacity_tokens(self) -> int:
        """Tokens the cache can hold when nothing is live (whole pages)."""
        return self.cache.n_pages * PAGE

    def truncate(self, slot: int, length: int) -> None:
        """Rolls a sequence back to its first `length` tokens; the next step continues from there
        (the reference's rollback of a conversation turn, src/conversation.rs:334-349 of
        yusiwen/minfer).  Refused for models with per-sequence state and once a windowed layer
        has given up pages the shorter sequence would need."""
        try:
            self.cache.truncate(slot, length)
        except CacheError as e:
            raise StepError(str(e)) from None

    def stop_tokens(self):
        """The model's own stop tokens: config.json's eos_token_id and, where the model folder has
        one, generation_config.json's (the reference stops on eos or <|im_end|>,
        src/main.rs:626-628 of yusiwen/minfer)."""
        return tuple(getattr(self.model, "stop_tokens", self.model.spec.stop_tokens))

    def decode_session(self, n_seqs: int, max_len: int, sampler, use_graph: bool = True):
        """A `DecodeSession` for this batch size, reused (with its captured graph) while the
        size, the reach (`max_len` rounded up to a power of two, at least 256, at most the model's
        positions) and the sampling options other than the seed stay the same.  At most
        MAX_SESSIONS are kept; the one unused for longest gives up its graph and buffers."""
        from .decode import DecodeSession
        reach = 256                          # in powers of two: prompts of many lengths share few captures
        while reach < max_len:
            reach *= 2
        max_len = min(self.max_positions, reach)
        key = (n_seqs, max_len, sampler.structure, use_graph)
        session = self._sessions.get(key)
        if session is None:
            while len(self._sessions) >= MAX_SESSIONS:
                _, old = self._sessions.popitem(last=False)
                old.release()
            session = self._sessions[key] = DecodeSession(self, n_seqs, max_len, sampler, use_graph)
        else:
            self._sessions.move_to_end(key)
        return session

    # ------------------------------------------------------------ one step
    def build_context(self, slots: Sequence[int], tokens: Sequence[Sequence[int]], want: Want) -> StepContext:
        """Checks the step, reserves its cache pages and uploads its metadata in one copy."""
        if len(slots) != len(tokens) or not slots:
            raise StepError("a step needs at least one sequence and as many token lists as slots")
        if len(set(slots)) != len(slots):
            raise StepError(f"a slot appears twice in one step: {list(slots)}")
        n_new = [len(t) for t in tokens]
        start, new_len = [], {}
        for b, (s, n) in enumerate(zip(slots, n_new)):
            if n < 1:
                raise StepError(f"sequence {b} (slot {s}) brings no tokens")
            try:
                cur = self.cache.length(s)
            except CacheError as e:
                raise StepError(str(e)) from None
            if cur + n > self.max_positions:
                raise StepError(f"sequence {b} (slot {s}): position {cur + n - 1} exceeds the model's "
                                f"{self.max_positions} positions")
            start.append(cur)
            new_len[s] = cur + n
        flat = np.fromiter((t for seq in tokens for t in seq), dtype=np.int64, count=sum(n_new))
        if flat.min() < 0 or flat.max() >= self.vocab_size:
            bad = int(flat[(flat < 0) | (flat >= self.vocab_size)][0])
            raise StepError(f"embedding id {bad} >= vocab {self.vocab_size}" if bad >= 0
                            else f"embedding id {bad} is negative")
        n_tok, n_seq = int(flat.size), len(slots)
        cu = np.zeros(n_seq + 1, dtype=np.int64)
        cu[1:] = np.cumsum(n_new)
        if isinstance(want, str):
            if want == "last":
                rows: Optional[np.ndarray] = cu[1:] - 1
            elif want == "all":
                rows = None
            else:
                raise StepError(f"want must be 'last', 'all' or per-sequence offsets, got {want!r}")
        else:
            if len(want) != n_seq:
                raise StepError("want needs one list of offsets per sequence")
            picked = []
            for b, offs in enumerate(want):
                for o in offs:
                    if not 0 <= int(o) < n_new[b]:
                        raise StepError(f"sequence {b}: wanted offset {o} outside its {n_new[b]} new tokens")
                    picked.append(cu[b] + int(o))
            rows = np.asarray(picked, dtype=np.int64)

        self.cache.reserve(new_len)          # CacheFull leaves everything as it was
        max_len = max(new_len.values())
        self.model.prepare(max_len)
        n_cols = (max_len + PAGE - 1) // PAGE
        seq_of_tok = np.repeat(np.arange(n_seq), n_new)
        positions = np.concatenate([np.arange(s, s + n) for s, n in zip(start, n_new)])
        pieces = [flat, positions, seq_of_tok, cu, np.asarray(start), np.asarray(slots),
                  rows if rows is not None else np.zeros(0, dtype=np.int64)]
        for g in self.cache.groups:
            pieces.append(np.asarray(self.cache.page_rows(g, slots, n_cols), dtype=np.int64).reshape(-1))
        packed = np.concatenate(pieces).astype(np.int32)
        dev = torch.from_numpy(packed).to(self.device)
        views, off = [], 0
        for p in pieces:
            views.append(dev[off:off + p.size])
            off += p.size
        tables = {id(g): views[7 + i].view(n_seq, n_cols) for i, g in enumerate(self.cache.groups)}
        ctx = StepContext(
            cache=self.cache, n_tokens=n_tok, n_seqs=n_seq, token_ids=views[0], positions=views[1],
            seq_of_tok=views[2], cu_seqlens=views[3], start_pos=views[4], slot_ids=views[5],
            logit_rows=None if rows is None else views[6], page_tables=tables, max_len=max_len,
            max_new=max(n_new), all_decode=all(n == 1 for n in n_new), host_new=n_new, host_start=start)
        ctx.new_lengths = new_len
        return ctx

    def step(self, slots: Sequence[int], tokens: Sequence[Sequence[int]], want: Want = "last") -> torch.Tensor:
        """Runs the given new tokens of each sequence (after what its slot already holds) and
        returns float32 logits `[wanted][vocab]`, ordered by sequence and then by offset.
        `want`: 'last' (each sequence's last new token), 'all', or offsets per sequence."""
        ctx = self.build_context(slots, tokens, want)
        logits = self.model.forward(ctx)
        self.cache.commit(ctx.new_lengths)
        return logits

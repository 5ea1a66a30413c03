"""Decode steps with everything that changes per step kept on the device, so that one step
(model, sampling, moving every sequence on by one) can be captured once as a HIP graph and
replayed.

The reference reuses its built graph across decode steps because positions are data, not
structure (src/graph/params.rs:39-52, src/graph/cache.rs:37-54 of yusiwen/minfer), and its
CUDA path captures the step as a CUDA graph (src/cuda.rs:480-527).  Here token ids,
positions, page tables, sampler counters and the recent-token windows live in buffers of a
fixed size per batch size; the host only reserves pages ahead and reads the sampled tokens,
and it may start the next step before it has read them (`launch` / `collect`).
"""
from __future__ import annotations

import gc
import weakref
from typing import Dict, List, Optional, Sequence

import torch

from ..cache.paged import PAGE
from ..kernels import ops, tuning
from ..sampling.params import REPEAT_LAST_N
from .batch import StepContext


class DecodeSession:
    """Buffers (and, once captured, the graph) for `n_seqs` sequences decoding up to
    `max_len` positions.  `bind` points it at a set of live sequences: which slots they live in,
    their page tables, their random streams (the sampling seed folded with each sequence's key)
    and their positions are all data in device buffers, so one captured step serves any set of
    sequences and any seed.  What is baked into a capture is the batch size, the reach and the
    sampling options other than the seed."""

    def __init__(self, engine, n_seqs: int, max_len: int, sampler, use_graph: bool = True):
        # the engine owns its sessions; the way back is a weak reference, so that an engine that
        # goes out of use is freed at once, with its graphs, and not whenever the collector of
        # reference cycles happens to run (which may be in the middle of another capture)
        self._engine = weakref.ref(engine)
        self.n, self.sampler = n_seqs, sampler
        self.max_len = max_len
        self.n_cols = (max_len + PAGE - 1) // PAGE
        self.use_graph = use_graph and engine.device.type == "cuda" and not tuning.DEBUG_SYNC
        dev = engine.device
        i32 = dict(dtype=torch.int32, device=dev)
        self.token_ids = torch.zeros(n_seqs, **i32)
        self.positions = torch.zeros(n_seqs, **i32)
        self.seq_of_tok = torch.arange(n_seqs, **i32)
        self.cu_seqlens = torch.arange(n_seqs + 1, **i32)
        self.slot_ids = torch.zeros(n_seqs, **i32)
        self.tables: Dict[int, torch.Tensor] = {
            id(g): torch.full((n_seqs, self.n_cols), -1, **i32) for g in engine.cache.groups}
        self.streams = torch.zeros(n_seqs, dtype=torch.int64, device=dev)
        self.steps = torch.zeros(n_seqs, **i32)
        self.sampled = torch.zeros(n_seqs, **i32)
        self.prev = torch.zeros((n_seqs, REPEAT_LAST_N), **i32)
        self.n_prev = torch.zeros(n_seqs, **i32)
        self.cursor = torch.zeros(n_seqs, **i32)
        # results of the two steps that may be in flight travel to pinned host memory
        self._pinned = self._events = None
        if dev.type == "cuda":
            self._pinned = [torch.empty(n_seqs, dtype=torch.int32, pin_memory=True) for _ in range(2)]
            self._events = [torch.cuda.Event() for _ in range(2)]
        self._host_out: List[Optional[List[int]]] = [None, None]
        self._launched = self._collected = 0
        self.last_logits: Optional[torch.Tensor] = None
        self.graph: Optional[torch.cuda.CUDAGraph] = None
        self._lease = None                   # ops.GraphLease of the captured graph
        self.warm = False
        self._finalizer = None
        self.slots: List[int] = []
        self._host_tables: Dict[int, List[List[int]]] = {}
        engine.model.prepare(max_len)

    @property
    def engine(self):
        engine = self._engine()
        if engine is None:
            raise RuntimeError("the engine of this decode session is gone")
        return engine

    # ------------------------------------------------------------ binding
    def abandon(self) -> None:
        """After an error: waits for whatever is in flight and forgets it, so the session can be
        bound again."""
        if self.engine.device.type == "cuda":
            torch.cuda.synchronize(self.engine.device)
        self._collected = self._launched

    def release(self) -> None:
        """Gives up the captured graph and with it the memory pool it holds."""
        self.graph = None
        self.warm = False
        if self._finalizer is not None:
            self._finalizer()                # gives the lease back (once)
        self._lease = self._finalizer = None

    def bind(self, slots: Sequence[int], next_tokens: Sequence[int], keys: Sequence[int],
             steps: Sequence[int], sampler=None) -> None:
        """The sequences in `slots` will each be fed `next_tokens[i]` at their current length.
        `keys[i]` names sequence i's random stream under the sampler's seed; `sampler` replaces
        the session's (same options, any seed)."""
        if sampler is not None:
            if sampler.structure != self.sampler.structure:
                raise ValueError("decode session bound with other sampling options than it was made for")
            self.sampler = sampler
        if len(slots) != self.n:
            raise ValueError(f"session is for {self.n} sequences, got {len(slots)}")
        cache, dev = self.engine.cache, self.engine.device
        self.slots = list(slots)
        lengths = [cache.length(s) for s in slots]
        self.token_ids.copy_(torch.tensor(list(next_tokens), dtype=torch.int32))
        self.positions.copy_(torch.tensor(lengths, dtype=torch.int32))
        self.slot_ids.copy_(torch.tensor(self.slots, dtype=torch.int32))
        self.streams.copy_(torch.tensor(self.sampler.streams(keys), dtype=torch.int64))
        self.steps.copy_(torch.tensor(list(steps), dtype=torch.int32))
        self._host_tables = {}
        if self._launched != self._collected:
            raise RuntimeError("decode session bound while a step is in flight")

    def set_windows(self, windows: Sequence[Sequence[int]]) -> None:
        """Recent tokens of each sequence for the penalties (at most the last 64)."""
        rows = [list(w)[-REPEAT_LAST_N:] for w in windows]
        flat = torch.zeros((self.n, REPEAT_LAST_N), dtype=torch.int32)
        for i, r in enumerate(rows):
            if r:
                flat[i, :len(r)] = torch.tensor(r, dtype=torch.int32)
        self.prev.copy_(flat)
        self.n_prev.copy_(torch.tensor([len(r) for r in rows], dtype=torch.int32))
        self.cursor.copy_(torch.tensor([len(r) % REPEAT_LAST_N for r in rows], dtype=torch.int32))

    # ------------------------------------------------------------ one step
    def _context(self) -> StepContext:
        return StepContext(
            cache=self.engine.cache, n_tokens=self.n, n_seqs=self.n, token_ids=self.token_ids,
            positions=self.positions, seq_of_tok=self.seq_of_tok, cu_seqlens=self.cu_seqlens,
            start_pos=self.positions, slot_ids=self.slot_ids, logit_rows=None, page_tables=self.tables,
            max_len=self.max_len, max_new=1, all_decode=True, host_new=[1] * self.n, host_start=None)

    def _run(self) -> None:
        logits = self.engine.model.forward(self._context())
        self.last_logits = logits          # float32 [n_seqs][vocab] of the step run last (penalties applied in place)
        self.sampler(logits, self.streams, self.steps, self.sampled, self.prev, self.n_prev)
        ops.advance(self.token_ids, self.sampled, self.positions, self.steps, self.prev, self.n_prev, self.cursor)

    def step(self) -> List[int]:
        """Runs one token of every bound sequence and returns the next sampled tokens."""
        return self.collect(self.launch())

    def launch(self) -> int:
        """Starts one step (the sampled token of the step before is fed back on the device) and
        returns its handle without waiting for it.  At most two steps may be outstanding, so
        the host can start step n + 1 before it has looked at the tokens of step n."""
        if self._launched - self._collected >= 2:
            raise RuntimeError("two decode steps are already in flight")
        cache = self.engine.cache
        new_len = {s: cache.length(s) + 1 for s in self.slots}
        if max(new_len.values()) > self.max_len:
            raise ValueError(f"decode session was sized for {self.max_len} positions")
        # A page table row changes only when its sequence starts a new page (or, in a windowed
        # group, gives one back): that is the only time the host touches the tables.
        grows = [s for s, n in new_len.items() if (n - 1) % PAGE == 0]
        windowed = any(g.request.window is not None for g in cache.groups)
        if grows:
            cache.reserve({s: new_len[s] for s in grows})
        if grows or windowed or not self._host_tables:
            for g in cache.groups:
                if self._host_tables and not grows and g.request.window is None:
                    continue
                rows = cache.page_rows(g, self.slots, self.n_cols)
                if self._host_tables.get(id(g)) != rows:
                    self.tables[id(g)].copy_(torch.tensor(rows, dtype=torch.int32))
                    self._host_tables[id(g)] = rows
        if self.graph is not None and self._lease.stale():
            self.release()                   # a buffer the graph points at was replaced: capture again, let the old one go
        if not self.use_graph:
            self._run()
        elif self.graph is not None:
            self.graph.replay()
        elif not self.warm:
            self._run()                      # first step runs eagerly: loads and sizes everything
            self.warm = True
        else:
            graph = torch.cuda.CUDAGraph()
            collecting = gc.isenabled()
            gc.disable()                     # nothing may be freed on the device while the stream is captured
            try:
                with torch.cuda.graph(graph):
                    self._run()
            finally:
                if collecting:
                    gc.enable()
            self.graph = graph
            self._lease = ops.lease_graph()
            self._finalizer = weakref.finalize(self, ops.release_graph, self._lease)
            graph.replay()
        k = self._launched % 2
        if self._pinned is not None:
            self._pinned[k].copy_(self.sampled, non_blocking=True)
            self._events[k].record()
        else:
            self._host_out[k] = self.sampled.cpu().tolist()
        cache.commit(new_len)
        self._launched += 1
        return self._launched - 1

    def collect(self, handle: int) -> List[int]:
        """The sampled tokens of a launched step, in the order of the bound sequences; steps are
        collected in the order they were launched."""
        if handle != self._collected or handle >= self._launched:
            raise RuntimeError(f"decode step {handle} is not the next one to collect")
        k = handle % 2
        if self._pinned is not None:
            self._events[k].synchronize()
            tokens = self._pinned[k].tolist()
        else:
            tokens = self._host_out[k]
        self._collected += 1
        return tokens

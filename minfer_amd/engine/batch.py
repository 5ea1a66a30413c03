"""The ragged batch of one step as the parts see it.

All sequences' new tokens are concatenated: token t belongs to sequence `seq_of_tok[t]`
(an index into the step's batch, not a slot) and sits at absolute position `positions[t]`;
it attends to its own sequence's cache rows up to that position and to nothing else.
Positions are data, never structure (src/graph/ops.rs:3-6 of yusiwen/minfer), and a step's
keys are stored before its attention reads them (src/graph/scheduler.rs:12-15).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch


@dataclass
class StepContext:
    cache: object                        # minfer_amd.cache.Cache
    n_tokens: int
    n_seqs: int
    token_ids: torch.Tensor              # int32 [n_tokens]
    positions: torch.Tensor              # int32 [n_tokens]
    seq_of_tok: torch.Tensor             # int32 [n_tokens]
    cu_seqlens: torch.Tensor             # int32 [n_seqs + 1], offsets of each sequence's tokens
    start_pos: torch.Tensor              # int32 [n_seqs], tokens each sequence held before the step
    slot_ids: torch.Tensor               # int32 [n_seqs], cache slot of each sequence
    logit_rows: Optional[torch.Tensor]   # int32 [n_wanted] rows of the step whose logits are wanted
    page_tables: Dict[int, torch.Tensor]  # id(group) -> int32 [n_seqs][n_cols]
    max_len: int                         # bound on position + 1 over the step's tokens
    max_new: int                         # longest run of new tokens of one sequence
    all_decode: bool                     # every sequence brings exactly one token
    # host copies of the ragged layout, for parts that plan their launches on the host.  Which
    # slot a sequence lives in is not among them: slots are addressed through `slot_ids` only.
    host_new: List[int] = field(default_factory=list)        # new tokens of each sequence
    host_start: Optional[List[int]] = None                   # tokens each held before (None in a decode step)
    new_lengths: Dict[int, int] = field(default_factory=dict)   # slot -> tokens held after the step
    # between a product that adds into the residual stream and the norm that reads it next (see
    # `parts.base.announce_norm`): the norm the running part's output meets, the norm that follows
    # the running block, and what a product prepared for the next norm
    norm_next: object = None
    norm_after_block: object = None
    norm_ahead: object = None
    _memo: Dict = field(default_factory=dict, repr=False)

    def page_table(self, group) -> torch.Tensor:
        return self.page_tables[id(group)]

    def query_tiles(self, block: int):
        """(tile_seq, tile_q0) int32 on the device: the blocks of `block` consecutive new
        tokens of each sequence, for kernels that give a workgroup to each.  Built from the
        host's copy of the step once and kept."""
        key = ("query_tiles", block)
        if key not in self._memo:
            tiles = []
            for b, n in enumerate(self.host_new):
                first = self.host_start[b] if self.host_start else 0
                for q0 in range(0, n, block):
                    tiles.append((first + min(q0 + block, n), b, q0))     # keys its last query sees
            tiles.sort(key=lambda t: -t[0])                               # longest first: they finish together
            seqs, starts = [t[1] for t in tiles], [t[2] for t in tiles]
            both = torch.tensor([seqs, starts], dtype=torch.int32).to(self.token_ids.device)
            self._memo[key] = (both[0], both[1])
        return self._memo[key]

    def shared_query_tiles(self, block: int, page: int, window: int, n_heads: int, n_cu: int, per_cu: int,
                           min_pages: int, max_shares: int, min_imbalance: float = 1.5):
        """(tile_seq, tile_q0, tile_share, n_slots, most shares): as `query_tiles`, but a block of queries with
        many pages of keys is listed several times, once for each of the workgroups that are to
        take its pages in turn.  A workgroup should get at most its even share of the step's pages
        (all blocks x `n_heads` heads over the `n_cu` x `per_cu` workgroups that run at once), and at
        least `min_pages`; entry i of tile_share is share + 256 * shares + 65536 * slot (0 for a
        block listed once), slots numbering the blocks that are shared.  None where no block needs
        sharing, or where sharing cannot gain: the step takes at least as long as a CU's even
        share of all pages and as its longest block, and only where the longest block is
        `min_imbalance` times that share is there time to win by cutting it (putting the parts
        together has a price).  Kept per set of arguments: layers with other head counts plan for
        themselves."""
        key = ("shared_query_tiles", block, page, window, n_heads, n_cu, per_cu, min_pages, max_shares, min_imbalance)
        if key not in self._memo:
            tiles = []
            for b, n in enumerate(self.host_new):
                first = self.host_start[b] if self.host_start else 0
                for q0 in range(0, n, block):
                    last_key = first + min(q0 + block, n) - 1
                    first_key = max(0, first + q0 - window + 1) if window > 0 else 0
                    tiles.append((last_key // page - first_key // page + 1, b, q0))
            total = sum(t[0] for t in tiles)
            longest = max(t[0] for t in tiles)
            if longest * max(1, n_cu) < min_imbalance * total * n_heads:
                self._memo[key] = None
                return None
            target = max(1, int(min_pages), -(-total * n_heads // max(1, n_cu * per_cu)))
            entries, n_slots, most = [], 0, 1
            for pages, b, q0 in tiles:
                shares = min(max_shares, (pages + target - 1) // target)
                most = max(most, shares)
                if shares <= 1:
                    entries.append((pages, b, q0, 0))
                    continue
                for s in range(shares):
                    entries.append(((pages - s + shares - 1) // shares, b, q0, s + 256 * shares + 65536 * n_slots))
                n_slots += 1
            if n_slots == 0:
                self._memo[key] = None
            else:
                entries.sort(key=lambda e: -e[0])                         # longest first
                cols = torch.tensor([[e[1] for e in entries], [e[2] for e in entries], [e[3] for e in entries]],
                                    dtype=torch.int32).to(self.token_ids.device)
                self._memo[key] = (cols[0], cols[1], cols[2], n_slots, most)
        return self._memo[key]

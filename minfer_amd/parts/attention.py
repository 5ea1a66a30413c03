"""Grouped-query attention over the cache.

norm'd x -> q,k,v = W x + b -> position encoding on q and k -> k,v stored at the tokens'
positions -> every query head h reads kv head h // (heads/kv_heads), rows 0..=position (or
the last `window` of them) -> softmax(q.k * scale) v -> W_o -> added to the residual
(src/models/qwen2/graph.rs:100-137, src/graph/cpu_backend.rs:437-494 of yusiwen/minfer).
q|k|v are one stacked matrix so a step reads one.
"""
from __future__ import annotations

import torch

from ..cache.paged import KVRequest
from ..kernels import ops
from ..weights.loader import TensorSpec
from .base import Mixer, POSITIONS, make_part, register_mixer
from .linear import Linear


@register_mixer("gqa_attention")
class GQAttention(Mixer):
    """params: hidden_size, n_heads, n_kv_heads, head_dim, scale, window (None or int),
    qkv_bias, out_bias, position (PartSpec), q/k/v/o (tensor name stems)."""

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        p = spec.params
        self.hidden, self.nh, self.nk, self.hd = (int(p[k]) for k in
                                                   ("hidden_size", "n_heads", "n_kv_heads", "head_dim"))
        self.scale = float(p["scale"])
        self.window = p.get("window")
        self.qkv_bias, self.out_bias = bool(p.get("qkv_bias", False)), bool(p.get("out_bias", False))
        self.names = {k: p[k] for k in ("q", "k", "v", "o")}
        if self.nh % self.nk:
            raise ValueError(f"gqa_attention: {self.nh} heads are not a multiple of {self.nk} kv heads")
        if self.hd % 16 or not 16 <= self.hd <= 256:
            raise ValueError(f"gqa_attention: head_dim {self.hd} is not supported by the attention "
                             "kernels (multiples of 16 from 16 to 256)")
        if self.window is not None and int(self.window) < 1:
            raise ValueError(f"gqa_attention: window {self.window} must be >= 1")
        self.position = make_part(POSITIONS, p["position"], rt, "position encoding")
        self.qkv = self.o = None

    def tensor_specs(self):
        n, s = self.names, {}
        for key, rows in (("q", self.nh * self.hd), ("k", self.nk * self.hd), ("v", self.nk * self.hd)):
            s[n[key] + ".weight"] = TensorSpec((rows, self.hidden))
            if self.qkv_bias:
                s[n[key] + ".bias"] = TensorSpec((rows,))
        s[n["o"] + ".weight"] = TensorSpec((self.hidden, self.nh * self.hd))
        if self.out_bias:
            s[n["o"] + ".bias"] = TensorSpec((self.hidden,))
        return s

    def load(self, get):
        n = self.names
        ws = [get(n[k] + ".weight") for k in ("q", "k", "v")]
        bs = [get(n[k] + ".bias") for k in ("q", "k", "v")] if self.qkv_bias else None
        self.qkv = Linear.stacked(ws, bs)
        self.o = Linear(get(n["o"] + ".weight"), get(n["o"] + ".bias") if self.out_bias else None)

    def cache_request(self):
        return KVRequest(self.nk, self.hd, None if self.window is None else int(self.window))

    def decode_copies(self, make: bool, min_row_length: int = 0) -> int:
        return self.qkv.decode_copy(make, min_row_length) + self.o.decode_copy(make, min_row_length)

    def prepare(self, max_len: int) -> None:
        self.position.prepare(max_len)

    takes_normed = True

    def forward(self, x, h, ctx, entry: int, writes_cache: bool) -> None:
        kc, vc, group = ctx.cache.kv(entry)
        table = ctx.page_table(group)
        qkv = self.qkv(x, out_dtype=torch.float32)
        window = 0 if self.window is None else int(self.window)
        o = torch.empty((x.shape[0], self.nh * self.hd), dtype=self.rt.dtype, device=x.device)
        tables = self.position.rotation_tables(ctx.max_len)
        if tables is not None and self.rt.is_bf16 and ctx.all_decode:
            # decode: rotation, cache write and attention in one kernel
            ops.attn_decode_rope(qkv, tables[0], tables[1], kc, vc, table, ctx.positions, ctx.seq_of_tok, o,
                                 self.nh, self.nk, self.hd, self.scale, window, ctx.max_len, writes_cache)
            self.o(o, out=h, accumulate=True, ctx=ctx)
            return
        q = torch.empty_like(o)
        if tables is not None:         # rotation and cache write in one kernel
            ops.rope_kvwrite(qkv, tables[0], tables[1], ctx.positions, ctx.seq_of_tok, table, q, kc, vc,
                             self.nh, self.nk, self.hd, writes_cache)
        else:                          # any other encoding: it treats q and k, the cache stores
            self.position.encode(qkv, ctx, self.nh, self.nk)
            if writes_cache:
                ctx.cache.store_kv(entry, qkv, ctx, self.nh, q)
            else:
                ops.rope_kvwrite(qkv, None, None, ctx.positions, ctx.seq_of_tok, table, q, None, None,
                                 self.nh, self.nk, self.hd, False)
        if self.rt.is_bf16 and not ctx.all_decode and ops.HAVE_PREFILL_ATTENTION:
            ops.attn_prefill(q, kc, vc, table, ctx, o, self.nh, self.nk, self.hd, self.scale, window)
        else:
            ops.attn_tokens(q, kc, vc, table, ctx.positions, ctx.seq_of_tok, o, self.nh, self.nk,
                            self.hd, self.scale, window, ctx.max_len)
        self.o(o, out=h, accumulate=True, ctx=ctx)

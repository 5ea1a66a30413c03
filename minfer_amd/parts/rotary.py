"""Half-split ("NeoX") rotary position encoding over the whole head: element i pairs with
i + head_dim/2, angle = position * freq_scale / theta^(2i/head_dim)
(src/graph/cpu_backend.rs:403-434 of yusiwen/minfer; q and k are rotated after their bias
and before the cache write, v is not, src/models/qwen2/graph.rs:100-113).  cos and sin come
from a table built once on the device in double precision.  The attention mixer takes the
tables and rotates inside its own kernels; `encode` is the plain form for any other user."""
from __future__ import annotations

from ..kernels import ops
from .base import PositionEncoding, register_position

# positions the table is first built for; it doubles from there up to the model's bound, and a
# table that covers the bound is never replaced (so a captured step's address stays good)
FIRST_TABLE = 4096


@register_position("rope_neox")
class RotaryNeoX(PositionEncoding):
    """params: head_dim, theta, max_positions, freq_scale (default 1)."""

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        p = spec.params
        self.head_dim, self.theta = int(p["head_dim"]), float(p["theta"])
        self.freq_scale = float(p.get("freq_scale", 1.0))
        self.max_positions = int(p["max_positions"])
        if self.head_dim % 2:
            raise ValueError(f"rope_neox: head_dim {self.head_dim} is odd")
        self.cos = self.sin = None
        self.generation = 0            # moves on when the table is replaced by a longer one

    def prepare(self, max_len: int) -> None:
        if max_len > self.max_positions:
            raise ValueError(f"position {max_len - 1} is beyond the model's {self.max_positions} positions")
        have = 0 if self.cos is None else self.cos.shape[0]
        if max_len > have:
            n = min(self.max_positions, max(FIRST_TABLE, 1 << (max_len - 1).bit_length()))
            if self.cos is not None:
                self.generation += 1
                ops.note_replaced_buffer(self.cos)
                ops.note_replaced_buffer(self.sin)
            self.cos, self.sin = ops.rope_table(n, self.head_dim // 2, self.theta, self.freq_scale,
                                                self.rt.device)

    def rotation_tables(self, max_len: int):
        self.prepare(max_len)
        return self.cos, self.sin

    def encode(self, qkv, ctx, n_heads: int, n_kv_heads: int) -> None:
        self.prepare(ctx.max_len)
        ops.rope_inplace(qkv, self.cos, self.sin, ctx.positions, n_heads + n_kv_heads,
                         n_heads + 2 * n_kv_heads, self.head_dim)

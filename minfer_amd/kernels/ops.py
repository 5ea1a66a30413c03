"""Python faces of the HIP kernels: each function checks its operands on the host (device,
type, shape, contiguity), then launches on torch's current stream.  Outputs are written
into tensors the caller allocated, so a captured step allocates nothing here except the
cached workspaces below.
"""
from __future__ import annotations

import ctypes
import sys
from ctypes import c_char_p, c_double, c_float, c_int, c_size_t, c_uint64, c_void_p
from typing import Dict, Optional, Tuple

import torch

from . import build, tuning
from ..cache.paged import v_page_shape

PAGE = 64          # tokens per cache page (MF_PAGE in csrc/common.h)
HAVE_PREFILL_ATTENTION = True
PREFILL_MAX_SHARES = 8  # workgroups that may take the pages of one block of queries of the prompt attention in turn
PREFILL_MIN_PAGES = 4   # ... each with at least this many pages
EPI_F32, EPI_ACC_F32, EPI_BF16, EPI_SWIGLU = 0, 1, 2, 3


class KernelError(RuntimeError):
    pass


_P = c_void_p
_PROTOTYPES = {
    "elementwise": {
        "mf_embed": [_P, c_int, _P, _P, c_int, c_int, c_int, _P],
        "mf_rmsnorm": [_P, _P, _P, _P, c_int, c_int, c_int, c_float, _P],
        "mf_gather_rows": [_P, _P, _P, c_int, c_int, _P],
        "mf_swiglu": [_P, c_int, _P, c_int, c_int, c_int, _P],
        "mf_convert": [_P, c_int, _P, c_int, c_size_t, _P],
        "mf_rope_table": [_P, _P, c_int, c_int, c_double, c_double, _P],
        "mf_rope_kvwrite": [_P, _P, _P, _P, _P, _P, c_int, _P, _P, _P, c_int, c_int, c_int, c_int,
                            c_int, c_int, _P],
        "mf_rope_inplace": [_P, _P, _P, _P, c_int, c_int, c_int, c_int, _P],
        "mf_fill_normal": [_P, c_int, c_size_t, c_uint64, c_float, c_int, _P],
    },
    "probe": {
        "mf_probe_read": [_P, c_size_t, _P, c_int, _P],
        "mf_probe_mfma": [c_int, _P, c_int, _P],
    },
    "host_random": {
        "mf_fill_normal_host": [_P, c_int, c_size_t, c_uint64, c_float, c_int, c_int],
    },
    "gemm_f32": {
        "mf_gemm_f32": [_P, c_int, _P, c_int, _P, _P, c_int, c_int, c_int, c_int, c_int, _P],
    },
    "gemm_bf16": {
        "mf_gemm_bf16": [_P, c_int, _P, c_int, _P, _P, c_int, c_int, c_int, c_int, c_int, c_int, _P],
        "mf_gemm_bf16_splitk": [_P, c_int, _P, c_int, _P, _P, c_int, _P, c_int, c_int, c_int, c_int, c_int, c_int,
                                c_int, _P],
        "mf_gemm_bf16_skinny": [_P, c_int, _P, _P, c_int, _P, _P, c_int, _P, c_int, c_int, c_int, c_int,
                                c_int, c_int, _P],
        "mf_gemm_bf16_normed": [_P, c_int, _P, _P, c_float, _P, _P, c_int, _P, _P, c_int, c_int, c_int, c_int,
                                c_int, _P],
        "mf_gemm_bf16_skinny_fused": [_P, c_int, _P, _P, c_int, _P, _P, c_int, _P, c_int, c_int, c_int, c_int,
                                      c_int, c_int, _P, c_int, c_float, _P, _P, _P, c_int, _P],
        "mf_gemm_bf16_plan": [c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_char_p, c_int],
        "mf_gemm_bf16_tile_plan": [c_int, c_int, c_int, c_int, c_int, c_int, _P],
    },
    "attn_tokens_f32": {
        "mf_attn_tokens_f32": [_P, _P, _P, _P, c_int, _P, _P, _P, _P, c_int, c_int, c_int, c_int,
                               c_float, c_int, c_int, c_int, _P],
    },
    "attn_decode_bf16": {
        "mf_attn_decode_bf16": [_P, _P, _P, _P, c_int, _P, _P, _P, _P, c_int, c_int, c_int, c_int,
                                c_float, c_int, c_int, c_int, _P],
        "mf_attn_decode_rope_bf16": [_P, _P, _P, _P, _P, _P, c_int, _P, _P, _P, _P, c_int, c_int, c_int,
                                     c_int, c_float, c_int, c_int, c_int, c_int, _P],
    },
    "attn_prefill_bf16": {
        "mf_attn_prefill_bf16": [_P, _P, _P, _P, c_int, _P, _P, _P, _P, _P, _P, _P, c_int, _P, c_int, c_int, c_int,
                                 c_int, c_int, c_int, c_float, c_int, _P],
        "mf_attn_prefill_part_floats": [c_int],
        "mf_attn_prefill_rows": [c_int],
        "mf_attn_prefill_per_cu": [c_int],
    },
    "sampling": {
        "mf_argmax": [_P, c_int, c_int, c_int, _P, _P, c_int, _P],
        "mf_sample": [_P, c_int, c_int, c_int, c_float, _P, _P, _P, _P, _P],
        "mf_penalties": [_P, c_int, c_int, c_int, _P, c_int, _P, c_float, c_float, c_float, _P],
        "mf_top_k": [_P, c_int, c_int, c_int, c_int, _P],
        "mf_top_p": [_P, c_int, c_int, c_int, c_float, _P],
        "mf_sample_filtered": [_P, c_int, c_int, c_int, c_int, c_float, c_float, _P, _P, _P, _P, _P, _P],
        "mf_advance": [_P, _P, _P, _P, c_int, _P, c_int, _P, _P, _P],
    },
}
_functions: Dict[str, object] = {}


def _fn(lib: str, name: str):
    f = _functions.get(name)
    if f is None:
        f = getattr(build.load(lib), name)
        f.argtypes = _PROTOTYPES[lib][name]
        f.restype = c_int
        _functions[name] = f
    return f


def _stream() -> c_void_p:
    return c_void_p(torch.cuda.current_stream().cuda_stream)


def _check(rc: int, what: str) -> None:
    """Raises on a launch error.  With MF_DEBUG_SYNC the stream is synchronised after every launch,
    so a fault inside a kernel is reported here, under the name of the launch that caused it
    (the reference's debug_sync, src/cuda.rs:378-395 of yusiwen/minfer)."""
    if rc != 0:
        raise KernelError(f"{what}: HIP error {rc}"
                          + (" (invalid argument: a size the kernel does not take)" if rc == 1 else ""))
    if _trace is not None:
        ev = torch.cuda.Event(enable_timing=True)
        ev.record()
        _trace.append((what, ev))
    if tuning.DEBUG_SYNC and not torch.cuda.is_current_stream_capturing():
        try:
            torch.cuda.current_stream().synchronize()
        except RuntimeError as e:
            raise KernelError(f"{what}: failed on the device: {e}") from None
        print(f"[minfer_amd] {what} OK", file=sys.stderr, flush=True)


def _ptr(t: Optional[torch.Tensor]) -> c_void_p:
    return c_void_p(0 if t is None else t.data_ptr())


# ------------------------------------------------------------------ per-launch timing
_trace: Optional[list] = None


def start_trace() -> None:
    """From here on every launch is followed by an event on the stream; `stop_trace` turns them
    into (launch name, microseconds) pairs.  The time of a launch is the time between the event
    behind the launch before it and its own, so the GPU must not run dry in between: queue
    enough work first (`probe_mfma`) that the host stays ahead."""
    global _trace
    first = torch.cuda.Event(enable_timing=True)
    first.record()
    _trace = [("", first)]


def stop_trace():
    global _trace
    events, _trace = _trace or [], None
    if len(events) < 2:
        return []
    events[-1][1].synchronize()
    return [(name, events[i - 1][1].elapsed_time(ev) * 1e3) for i, (name, ev) in enumerate(events) if i]


def _need(t: torch.Tensor, name: str, dtype=None, shape=None) -> None:
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise KernelError(f"{name}: must be a tensor on the GPU (there is no CPU path)")
    if not t.is_contiguous():
        raise KernelError(f"{name}: must be contiguous, got strides {t.stride()} for shape {tuple(t.shape)}")
    if dtype is not None:
        ok = t.dtype in dtype if isinstance(dtype, (tuple, list)) else t.dtype == dtype
        if not ok:
            raise KernelError(f"{name}: dtype {t.dtype}, expected {dtype}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise KernelError(f"{name}: shape {tuple(t.shape)}, expected {tuple(shape)}")


def _is_bf16(t: torch.Tensor) -> int:
    return 1 if t.dtype == torch.bfloat16 else 0


_FLOATS = (torch.float32, torch.bfloat16)

# ------------------------------------------------------------------ workspaces
# Scratch buffers are shared by all callers and replaced by larger ones on demand.  A captured
# graph holds the addresses of the buffers that were current when it was captured, so an outgrown
# buffer must stay allocated while such a graph may still be replayed.  One rule, kept here: whoever
# captures ops calls takes a `GraphLease` right after the capture and gives it back when the
# graph is dropped (`lease_graph`, `release_graph`); a buffer that is replaced is kept while any
# lease is older than its replacement, and freed otherwise.  `lease.stale()` tells an owner that
# a buffer was replaced since its capture: it may capture again (and so let the old one go), or go
# on replaying, which stays safe.
_workspaces: Dict[Tuple[str, int], torch.Tensor] = {}
_counters: Dict[Tuple[str, int], torch.Tensor] = {}
_workspace_generation = 0
_retired: list = []                  # (generation in which the buffer was last current, buffer)
_leases: Dict[int, "GraphLease"] = {}
_next_lease = 0


def _device_index(device) -> int:
    dev = torch.device(device)
    if dev.type != "cuda":
        return -1
    return dev.index if dev.index is not None else torch.cuda.current_device()


class GraphLease:
    """Held by the owner of a captured graph for as long as the graph may be replayed."""

    def __init__(self, token: int, generation: int):
        self.token, self.generation = token, generation

    def stale(self) -> bool:
        """A buffer whose address the graph may hold has been replaced since the capture."""
        return self.generation != _workspace_generation


def lease_graph() -> GraphLease:
    """To be called right after a capture that recorded ops calls."""
    global _next_lease
    _next_lease += 1
    lease = _leases[_next_lease] = GraphLease(_next_lease, _workspace_generation)
    return lease


def release_graph(lease: Optional[GraphLease]) -> None:
    """The graph is gone: buffers that only it could still address are freed."""
    if lease is not None and _leases.pop(lease.token, None) is not None:
        _drop_unreachable()


def _drop_unreachable() -> None:
    oldest = min((l.generation for l in _leases.values()), default=None)
    _retired[:] = [(g, b) for g, b in _retired if oldest is not None and oldest <= g]


def _retire(buffer: torch.Tensor) -> None:
    """`buffer` is being replaced: the generation moves on, and the buffer stays allocated if a
    leased graph was captured while it was current."""
    global _workspace_generation
    _retired.append((_workspace_generation, buffer))
    _workspace_generation += 1
    _drop_unreachable()


def workspace(tag: str, n_floats: int, device) -> torch.Tensor:
    """A float32 scratch tensor of at least n_floats, kept per (tag, device) and replaced by one at
    least twice as large when it is outgrown.  Kernels that use one run in stream order, so sharing
    it is safe."""
    key = (tag, _device_index(device))
    w = _workspaces.get(key)
    if w is None or w.numel() < n_floats:
        if w is not None:
            _retire(w)
            n_floats = max(n_floats, 2 * w.numel())
        w = torch.empty(max(n_floats, 1 << 16), dtype=torch.float32, device=device)
        _workspaces[key] = w
    return w


def _zeroed_counters(tag: str, n: int, device) -> torch.Tensor:
    """int32 counters for kernels whose workgroups count themselves in and leave the counters at
    zero again: zero when made, kept per (tag, device), replaced (see above) when more are needed."""
    key = (tag, _device_index(device))
    c = _counters.get(key)
    if c is None or c.numel() < n:
        if c is not None:
            _retire(c)
            n = max(n, 2 * c.numel())
        c = torch.zeros(max(n, 1024), dtype=torch.int32, device=torch.device(device))
        _counters[key] = c
    return c


def workspace_generation() -> int:
    return _workspace_generation


def note_replaced_buffer(old: Optional[torch.Tensor] = None) -> None:
    """For any other buffer whose address a captured graph may hold (a rotation table that was
    rebuilt longer): `old` is treated like an outgrown workspace."""
    _retire(old if old is not None else torch.empty(0))


# ------------------------------------------------------------------ element-wise
def embed(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor) -> None:
    _need(table, "embed.table", _FLOATS)
    _need(ids, "embed.ids", torch.int32)
    n, d = ids.numel(), table.shape[1]
    _need(out, "embed.out", torch.float32, (n, d))
    _check(_fn("elementwise", "mf_embed")(_ptr(table), _is_bf16(table), _ptr(ids), _ptr(out), n, d,
                                           table.shape[0], _stream()), "embed")


def rmsnorm(x: torch.Tensor, weight: Optional[torch.Tensor], eps: float, out: torch.Tensor,
            row_idx: Optional[torch.Tensor] = None) -> None:
    _need(x, "rmsnorm.x", torch.float32)
    d = x.shape[-1]
    rows = out.shape[0]
    _need(out, "rmsnorm.out", _FLOATS, (rows, d))
    if weight is not None:
        _need(weight, "rmsnorm.weight", torch.float32, (d,))
    if row_idx is not None:
        _need(row_idx, "rmsnorm.row_idx", torch.int32, (rows,))
    elif x.shape[0] != rows:
        raise KernelError(f"rmsnorm: x has {x.shape[0]} rows, out has {rows}")
    _check(_fn("elementwise", "mf_rmsnorm")(_ptr(x), _ptr(row_idx), _ptr(weight), _ptr(out),
                                             _is_bf16(out), rows, d, float(eps), _stream()), "rmsnorm")


def gather_rows(x: torch.Tensor, idx: torch.Tensor, out: torch.Tensor) -> None:
    _need(x, "gather_rows.x", torch.float32)
    _need(idx, "gather_rows.idx", torch.int32)
    _need(out, "gather_rows.out", torch.float32, (idx.numel(), x.shape[1]))
    _check(_fn("elementwise", "mf_gather_rows")(_ptr(x), _ptr(idx), _ptr(out), idx.numel(),
                                                 x.shape[1], _stream()), "gather_rows")


def swiglu(gate_up: torch.Tensor, out: torch.Tensor) -> None:
    _need(gate_up, "swiglu.gate_up", _FLOATS)
    rows, two_nf = gate_up.shape
    if two_nf % 2:
        raise KernelError(f"swiglu: gate_up has an odd width {two_nf}")
    _need(out, "swiglu.out", _FLOATS, (rows, two_nf // 2))
    if _is_bf16(gate_up) and not _is_bf16(out):
        raise KernelError("swiglu: bfloat16 input with float32 output is not provided")
    _check(_fn("elementwise", "mf_swiglu")(_ptr(gate_up), _is_bf16(gate_up), _ptr(out), _is_bf16(out),
                                            rows, two_nf // 2, _stream()), "swiglu")


def convert(src: torch.Tensor, dst: torch.Tensor) -> None:
    _need(src, "convert.src", _FLOATS)
    _need(dst, "convert.dst", _FLOATS)
    if src.numel() != dst.numel() or src.dtype == dst.dtype:
        raise KernelError("convert: needs equal sizes and different types")
    _check(_fn("elementwise", "mf_convert")(_ptr(src), _is_bf16(src), _ptr(dst), _is_bf16(dst),
                                             src.numel(), _stream()), "convert")


def fill_normal(out: torch.Tensor, seed: int, std: float, round_bf16: bool = True) -> None:
    """N(0, std) values that depend on (seed, index) only, the same bits as `fill_normal_host`
    gives.  `round_bf16`: a float32 tensor gets values that bfloat16 represents."""
    _need(out, "fill_normal.out", _FLOATS)
    _check(_fn("elementwise", "mf_fill_normal")(_ptr(out), _is_bf16(out), out.numel(),
                                                 seed & 0xFFFFFFFFFFFFFFFF, float(std), 1 if round_bf16 else 0,
                                                 _stream()), "fill_normal")


def fill_normal_host(out: torch.Tensor, seed: int, std: float, round_bf16: bool = True, threads: int = 0) -> None:
    """The same fill into a CPU tensor (host code only; no GPU is touched)."""
    import os
    if not isinstance(out, torch.Tensor) or out.is_cuda or not out.is_contiguous() or out.dtype not in _FLOATS:
        raise KernelError("fill_normal_host: needs a contiguous float32 or bfloat16 tensor on the CPU")
    threads = threads or max(1, min(16, os.cpu_count() or 1))
    rc = _fn("host_random", "mf_fill_normal_host")(c_void_p(out.data_ptr()), _is_bf16(out), out.numel(),
                                                    seed & 0xFFFFFFFFFFFFFFFF, float(std),
                                                    1 if round_bf16 else 0, threads)
    if rc != 0:
        raise KernelError(f"fill_normal_host: error {rc}")


def rope_table(n_pos: int, half: int, theta: float, freq_scale: float, device):
    cs = torch.empty((n_pos, half), dtype=torch.float32, device=device)
    sn = torch.empty((n_pos, half), dtype=torch.float32, device=device)
    _need(cs, "rope_table.out")
    _check(_fn("elementwise", "mf_rope_table")(_ptr(cs), _ptr(sn), n_pos, half, float(theta),
                                                float(freq_scale), _stream()), "rope_table")
    return cs, sn


def rope_inplace(qkv: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, positions: torch.Tensor,
                 n_rot_heads: int, n_heads_total: int, head_dim: int) -> None:
    """The half-split rotation alone: the first `n_rot_heads` heads of every token's
    `[n_heads_total][head_dim]` row of 32-bit values are rotated in place."""
    n_tok = positions.numel()
    _need(qkv, "rope_inplace.qkv", torch.float32, (n_tok, n_heads_total * head_dim))
    _need(cos, "rope_inplace.cos", torch.float32)
    _need(sin, "rope_inplace.sin", torch.float32, tuple(cos.shape))
    if cos.shape[1] != head_dim // 2 or head_dim % 2 or n_rot_heads > n_heads_total:
        raise KernelError(f"rope_inplace: table {tuple(cos.shape)}, head_dim {head_dim}, {n_rot_heads} of {n_heads_total} heads")
    _need(positions, "rope_inplace.positions", torch.int32, (n_tok,))
    _check(_fn("elementwise", "mf_rope_inplace")(_ptr(qkv), _ptr(cos), _ptr(sin), _ptr(positions), n_tok,
                                                  n_rot_heads, n_heads_total, head_dim, _stream()), "rope_inplace")


def rope_kvwrite(qkv: torch.Tensor, cos: Optional[torch.Tensor], sin: Optional[torch.Tensor],
                 positions: torch.Tensor, seq_of_tok: torch.Tensor, page_table: torch.Tensor, q_out: torch.Tensor,
                 kcache: Optional[torch.Tensor], vcache: Optional[torch.Tensor], n_heads: int,
                 n_kv_heads: int, head_dim: int, write_kv: bool = True) -> None:
    """Rotates q and k, and stores k and v of the tokens at their positions in the cache pages
    (`v_page_shape` says how V lies in a page).  Without tables (cos and sin None) nothing is
    rotated: q is rounded into q_out and k, v are stored as they come."""
    n_tok = positions.numel()
    _need(qkv, "rope.qkv", torch.float32, (n_tok, (n_heads + 2 * n_kv_heads) * head_dim))
    if (cos is None) != (sin is None):
        raise KernelError("rope: cos and sin come together or not at all")
    if cos is not None:
        _need(cos, "rope.cos", torch.float32)
        _need(sin, "rope.sin", torch.float32, tuple(cos.shape))
        if cos.shape[1] != head_dim // 2:
            raise KernelError(f"rope: table has {cos.shape[1]} frequencies, head_dim {head_dim} needs {head_dim // 2}")
    _need(positions, "rope.positions", torch.int32, (n_tok,))
    _need(seq_of_tok, "rope.seq_of_tok", torch.int32, (n_tok,))
    _need(page_table, "rope.page_table", torch.int32)
    _need(q_out, "rope.q_out", _FLOATS, (n_tok, n_heads * head_dim))
    if write_kv:
        _need_caches("rope", kcache, vcache, q_out.dtype, n_kv_heads, head_dim)
    _check(_fn("elementwise", "mf_rope_kvwrite")(
        _ptr(qkv), _ptr(cos), _ptr(sin), _ptr(positions), _ptr(seq_of_tok), _ptr(page_table),
        page_table.shape[1], _ptr(q_out), _ptr(kcache if write_kv else None),
        _ptr(vcache if write_kv else None), _is_bf16(q_out), n_tok, n_heads, n_kv_heads, head_dim,
        1 if write_kv else 0, _stream()), "rope_kvwrite")


# ------------------------------------------------------------------ matrix products
_CU_COUNT: Optional[int] = None


def cu_count() -> int:
    """Compute units of the current device (256 on MI355X)."""
    global _CU_COUNT
    if _CU_COUNT is None:
        _CU_COUNT = int(torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count)
    return _CU_COUNT


# K = 256 NS for which the register-resident decode product is instantiated
# (MF_STATIONARY_NS in csrc/gemm_bf16.hip; `plan_linear` asks the library itself)
STATIONARY_NS = (4, 6, 8, 10, 12, 14, 16, 20, 24, 28, 32)
STATIONARY_K7 = 896      # and this K, which runs as seven waves of four steps (the narrowest model of the family)


def stationary_shape(n: int, k: int, folded: bool = False) -> bool:
    """True where the register-resident decode product is built for [n][k] weights (aligned
    operands given): K = 256 NS for one of the NS above, or 896, and at least 128 tiles of 16 weight rows;
    a K above 5120 only with a norm or SwiGLU folded in (`folded`)."""
    if k == STATIONARY_K7:
        return (n + 15) // 16 >= 64
    return k % 256 == 0 and k // 256 in STATIONARY_NS and (n + 15) // 16 >= 128 and (k <= 5120 or folded)


def skinny_plan(m: int, n: int, k: int, target_blocks: Optional[int] = None,
                swiglu: bool = False, tiled: bool = False) -> Tuple[int, int]:
    """(splits, k_per_split) of a product with at most 64 rows.  One split: one kernel, K divided
    between the waves of a block.  More: blocks of 128 weight rows with the activations staged in
    LDS, K split so that there is about one block per CU, and a second kernel that adds the parts.

    At most 16 rows take the one-kernel form, except against a K of 8192 and more that the
    register-resident kernel does not hold, where it does badly from 9 rows on (every block reads
    its own copy of the activations from L2; from 13 rows on where it reads the tiled copy of the
    weights: the down product of the 7B shape at 12 rows 28.9 us against 29.9, at 16 rows 32.4
    against 30.4) and where a CU's share of the weight rows fills its 16-row tiles poorly, unless
    the matrix is small (the down product of the 3B shape, 2048 x 11008, at 8 rows: 13.5 us in one
    kernel, half-filled tiles and all, against 15.0 in two; at 16 rows 17.1 against 15.4)."""
    if target_blocks is None:
        target_blocks = tuning.SKINNY_TARGET or cu_count()
    if m <= 16:
        share = (n + target_blocks - 1) // target_blocks          # weight rows of a block in the one-kernel form
        fill = share / float((share + 15) // 16 * 16)
        small = m <= 8 and n * k <= 24 << 20          # up to 48 MB of weights: the second kernel's few microseconds count
        if k < 8192 or (m <= (12 if tiled else 8) and fill >= 0.8) or small or stationary_shape(n, k, swiglu):
            return 1, (k + 255) // 256 * 256
    n_blocks = (n + 127) // 128
    chunks = (k + 255) // 256
    splits = max(1, min(chunks, target_blocks // max(1, n_blocks)))
    per = (chunks + splits - 1) // splits
    return (chunks + per - 1) // per, per * 256


def tile_plan(m: int, n: int, k: int, epi: int, aligned: bool = True, n_cu: Optional[int] = None) -> Tuple[int, int, int]:
    """(variant, splits, k_per_split) of a bfloat16 product of more than 64 rows, as the library
    chooses among its tile kernels (an estimate of the rounds their tiles take over the CUs); with
    splits > 1, K is cut over blocks and a second kernel adds the parts."""
    out = (c_int * 3)()
    rc = _fn("gemm_bf16", "mf_gemm_bf16_tile_plan")(m, n, k, 1 if aligned else 0, epi, n_cu or cu_count(), out)
    if rc != 0:
        raise KernelError(f"tile_plan: error {rc} for m {m}, n {n}, k {k}")
    return out[0], out[1], out[2]


def _k_split(m: int, n: int, k: int, swiglu: bool, aligned: bool, n_cu: Optional[int] = None,
             tiled: bool = False) -> Tuple[int, int]:
    """(splits, k_per_split) as `linear` and `linear_swiglu` cut a bfloat16 product of at most 64 rows."""
    target = tuning.SKINNY_TARGET or n_cu
    return skinny_plan(m, n, k, target_blocks=target, swiglu=swiglu, tiled=tiled)


def plan_linear(m: int, n: int, k: int, swiglu: bool = False, normed: bool = False, aligned: bool = True,
                out_bf16: bool = False, accumulate: bool = False, n_cu: Optional[int] = None,
                tiled: bool = False) -> Dict[str, object]:
    """Which kernel `linear` / `linear_swiglu` / `linear_normed` runs for a bfloat16 product of
    `m` rows against `[n][k]` weights, as the library itself decides it, without launching
    anything: {'kernel': name, 'splits': s, 'k_per_split': per}.  With `normed` an empty name
    means that no kernel folds the norm in at this shape (norm and product then run one after
    the other).  `n` counts the interleaved gate|up rows for `swiglu`; `tiled`: the product is
    given the tiled copy of the weights (it moves the row count from which K is cut over blocks)."""
    n_cu = n_cu or cu_count()
    epi = EPI_SWIGLU if swiglu else (EPI_BF16 if out_bf16 else (EPI_ACC_F32 if accumulate else EPI_F32))
    splits, per = 1, k
    if normed:
        if m > 16 or tuning.NO_FOLD:
            return dict(kernel="", splits=1, k_per_split=k)
    elif m <= 64:
        splits, per = _k_split(m, n, k, swiglu, aligned, n_cu, tiled)
    else:
        _, splits, per = tile_plan(m, n, k, epi, aligned, n_cu)
    name = ctypes.create_string_buffer(64)
    rc = _fn("gemm_bf16", "mf_gemm_bf16_plan")(m, n, k, 1 if aligned else 0, epi, splits, per,
                                               1 if normed else 0, n_cu, name, 64)
    if rc != 0:
        raise KernelError(f"plan_linear: error {rc} for m {m}, n {n}, k {k}")
    return dict(kernel=name.value.decode(), splits=splits, k_per_split=per)


def tile_weight(weight: torch.Tensor) -> torch.Tensor:
    """The tiled copy of a bfloat16 `[n][k]` matrix, k a multiple of 32: `[ceil(n / 16)][k / 32][16][32]`,
    rows padded with zeros to a multiple of 16.  The products of at most 64 rows read their
    weights a tile (a contiguous kilobyte) per wave and step from it; made once, when a model is
    loaded, where memory allows a second copy."""
    _need(weight, "tile_weight.weight", torch.bfloat16)
    n, k = weight.shape
    if k % 32:
        raise KernelError(f"tile_weight: k {k} is not a multiple of 32")
    n16 = (n + 15) // 16 * 16
    if n16 != n:
        weight = torch.cat([weight, torch.zeros((n16 - n, k), dtype=weight.dtype, device=weight.device)])
    return weight.view(n16 // 16, 16, k // 32, 32).permute(0, 2, 1, 3).contiguous()


def _need_tiled(tiled: Optional[torch.Tensor], name: str, n: int, k: int) -> None:
    if tiled is not None:
        _need(tiled, name, torch.bfloat16, ((n + 15) // 16, k // 32, 16, 32))


def linear(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
           accumulate: bool = False, variant: int = 0, tiled: Optional[torch.Tensor] = None) -> None:
    """out (+)= x @ weight^T (+ bias).  weight is [out][in].  float32 weights take the true
    32-bit kernel; bfloat16 weights take the matrix-core kernels (a few rows: the streaming
    kernel).  `out` is float32, or bfloat16 for a bfloat16 product that is stored.  `tiled`:
    `tile_weight(weight)`, which the kernels for at most 64 rows read instead where they can."""
    _need(x, "linear.x", _FLOATS)
    _need(weight, "linear.weight", x.dtype)
    m, k = x.shape
    n = weight.shape[0]
    if weight.shape[1] != k:
        raise KernelError(f"linear: x is [{m},{k}], weight is {tuple(weight.shape)}")
    _need(out, "linear.out", _FLOATS, (m, n))
    if bias is not None:
        _need(bias, "linear.bias", torch.float32, (n,))
    if m == 0:
        return
    if x.dtype == torch.float32:
        _need(out, "linear.out", torch.float32)
        _check(_fn("gemm_f32", "mf_gemm_f32")(_ptr(x), k, _ptr(weight), k, _ptr(bias), _ptr(out), n, m,
                                               n, k, 1 if accumulate else 0, _stream()), f"gemm_f32 {m}x{n}x{k}")
        return
    if accumulate and out.dtype != torch.float32:
        raise KernelError("linear: accumulation needs a float32 output")
    epi = EPI_BF16 if out.dtype == torch.bfloat16 else (EPI_ACC_F32 if accumulate else EPI_F32)
    aligned = not (x.data_ptr() % 16 or weight.data_ptr() % 16 or k % 8)
    if m <= 64 and variant == 0:
        splits, per = _k_split(m, n, k, False, aligned, tiled=tiled is not None)
        part = workspace("skinny", splits * m * n, x.device) if splits > 1 else None
        _need_tiled(tiled, "linear.tiled", n, k)
        _check(_fn("gemm_bf16", "mf_gemm_bf16_skinny")(_ptr(x), k, _ptr(weight), _ptr(tiled), k, _ptr(bias),
                                                        _ptr(out), n, _ptr(part), m, n, k, splits, per,
                                                        epi, _stream()), f"gemm_bf16_skinny {m}x{n}x{k}")
        return
    if variant == 0:
        variant, splits, per = tile_plan(m, n, k, epi, aligned)
        if splits > 1:
            part = workspace("skinny", splits * m * n, x.device)
            _check(_fn("gemm_bf16", "mf_gemm_bf16_splitk")(_ptr(x), k, _ptr(weight), k, _ptr(bias), _ptr(out), n,
                                                            _ptr(part), m, n, k, splits, per, epi, variant,
                                                            _stream()), f"gemm_bf16_splitk {m}x{n}x{k}")
            return
    _check(_fn("gemm_bf16", "mf_gemm_bf16")(_ptr(x), k, _ptr(weight), k, _ptr(bias), _ptr(out), n, m,
                                             n, k, epi, variant, _stream()), f"gemm_bf16 {m}x{n}x{k}")


def interleave_gate_up(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """Rows of gate and up `[nf][k]` in groups of 64: 32 gate rows, then the 32 up rows of the
    same outputs; the last group is padded with zero rows.  The layout `linear_swiglu` reads."""
    nf, k = gate.shape
    groups = (nf + 31) // 32
    pad = groups * 32 - nf
    if pad:
        z = torch.zeros((pad, k), dtype=gate.dtype, device=gate.device)
        gate, up = torch.cat([gate, z]), torch.cat([up, z])
    return torch.stack([gate.view(groups, 32, k), up.view(groups, 32, k)], dim=1).reshape(groups * 64, k).contiguous()


def linear_swiglu(x: torch.Tensor, weight: torch.Tensor, out: torch.Tensor, variant: int = 0,
                  tiled: Optional[torch.Tensor] = None) -> None:
    """out = silu(x @ Wg^T) * (x @ Wu^T) in one kernel; `weight` is `interleave_gate_up(Wg, Wu)`,
    everything bfloat16, `out` is [rows][nf].  `tiled`: `tile_weight(weight)`."""
    _need(x, "linear_swiglu.x", torch.bfloat16)
    _need(weight, "linear_swiglu.weight", torch.bfloat16)
    m, k = x.shape
    n = weight.shape[0]
    nf = out.shape[1]
    if weight.shape[1] != k or n % 64 or not n // 2 - 32 < nf <= n // 2:
        raise KernelError(f"linear_swiglu: x {tuple(x.shape)}, weight {tuple(weight.shape)}, out {tuple(out.shape)}")
    _need(out, "linear_swiglu.out", torch.bfloat16, (m, nf))
    if m == 0:
        return
    aligned = not (x.data_ptr() % 16 or weight.data_ptr() % 16 or k % 8)
    if m <= 64 and variant == 0:
        splits, per = _k_split(m, n, k, True, aligned, tiled=tiled is not None)
        part = workspace("skinny", splits * m * n, x.device) if m > 16 or splits > 1 else None
        _need_tiled(tiled, "linear_swiglu.tiled", n, k)
        _check(_fn("gemm_bf16", "mf_gemm_bf16_skinny")(_ptr(x), k, _ptr(weight), _ptr(tiled), k, _ptr(None), _ptr(out), nf,
                                                        _ptr(part), m, n, k, splits, per, EPI_SWIGLU, _stream()),
               f"gemm_bf16_skinny(swiglu) {m}x{n}x{k}")
        return
    if variant == 0:
        variant, splits, per = tile_plan(m, n, k, EPI_SWIGLU, aligned)
        if splits > 1:
            part = workspace("skinny", splits * m * n, x.device)
            _check(_fn("gemm_bf16", "mf_gemm_bf16_splitk")(_ptr(x), k, _ptr(weight), k, _ptr(None), _ptr(out), nf,
                                                            _ptr(part), m, n, k, splits, per, EPI_SWIGLU, variant,
                                                            _stream()), f"gemm_bf16_splitk(swiglu) {m}x{n}x{k}")
            return
    _check(_fn("gemm_bf16", "mf_gemm_bf16")(_ptr(x), k, _ptr(weight), k, _ptr(None), _ptr(out), nf, m, n, k,
                                             EPI_SWIGLU, variant, _stream()), f"gemm_bf16(swiglu) {m}x{n}x{k}")


NOT_BUILT = -2      # an entry point's answer for a shape it has no kernel for; nothing was launched


def linear_normed(x: torch.Tensor, norm_weight: torch.Tensor, eps: float, row_idx: Optional[torch.Tensor],
                  weight: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
                  accumulate: bool = False, swiglu: bool = False, tiled: Optional[torch.Tensor] = None) -> bool:
    """out (+)= rmsnorm(x[row_idx]) @ weight^T (+ bias) in one kernel, for the few-row shapes
    the register-resident decode product covers; with `swiglu`, `weight` is
    `interleave_gate_up(Wg, Wu)` and out = silu(gate) * up.  x is the float32 residual stream,
    weight bfloat16.  Returns False, having done nothing, when there is no such kernel for
    the shape: the caller then norms and multiplies in two steps.  `tiled`: `tile_weight(weight)`."""
    _need(x, "linear_normed.x", torch.float32)
    _need(weight, "linear_normed.weight", torch.bfloat16)
    k = x.shape[1]
    n = weight.shape[0]
    m = x.shape[0] if row_idx is None else row_idx.numel()
    if weight.shape[1] != k:
        raise KernelError(f"linear_normed: x is {tuple(x.shape)}, weight is {tuple(weight.shape)}")
    _need(norm_weight, "linear_normed.norm_weight", torch.float32, (k,))
    if row_idx is not None:
        _need(row_idx, "linear_normed.row_idx", torch.int32)
    if bias is not None:
        _need(bias, "linear_normed.bias", torch.float32, (n,))
    if swiglu:
        nf = out.shape[1]
        if n % 64 or not n // 2 - 32 < nf <= n // 2 or bias is not None or accumulate:
            raise KernelError(f"linear_normed(swiglu): weight {tuple(weight.shape)}, out {tuple(out.shape)}")
        _need(out, "linear_normed.out", torch.bfloat16, (m, nf))
        epi, ldc = EPI_SWIGLU, nf
    else:
        _need(out, "linear_normed.out", _FLOATS, (m, n))
        if accumulate and out.dtype != torch.float32:
            raise KernelError("linear_normed: accumulation needs a float32 output")
        epi = EPI_BF16 if out.dtype == torch.bfloat16 else (EPI_ACC_F32 if accumulate else EPI_F32)
        ldc = n
    if m == 0:
        return True
    if m > 16 or tuning.NO_FOLD:
        return False
    _need_tiled(tiled, "linear_normed.tiled", n, k)
    rc = _fn("gemm_bf16", "mf_gemm_bf16_normed")(_ptr(x), k, _ptr(row_idx), _ptr(norm_weight), float(eps),
                                                 _ptr(weight), _ptr(tiled), k, _ptr(bias), _ptr(out), ldc, m, n, k,
                                                 epi, _stream())
    if rc == NOT_BUILT:
        return False
    _check(rc, f"gemm_bf16_normed{'(swiglu)' if swiglu else ''} {m}x{n}x{k}")
    return True


NORM_SUM_RUN = 256       # columns a partial sum of squares covers (a block of the kernel that adds a K split's parts)


# Steps of at most 16 rows prepare the next norm in a product's epilogue only for rows of this many
# values: measured at batch 8 (a decode step with it against without), width 896: 10 % slower (the
# reading product waits for the rows' sums, a trip to memory, where the whole kernel is 7 us), 1536
# and 2048: 0.5 % slower, 3584: 0.7 % faster (2.4 % at batch 1), 5120: 4.5 % faster; from 5121 on
# the register-resident product has no form that reads bfloat16 activations.
NORM_AHEAD_16_WIDTHS = (3072, 5120)


def norm_sum_parts(n: int, m: int = 64) -> int:
    """Partial sums of squares a row of `n` values comes with from a product of `m` rows (see
    `linear_fused`): one per run of 256 columns from 17 rows on (the kernel that adds the parts of a K
    split writes them), one per workgroup of the product's one kernel for at most 16 rows."""
    runs = (n + NORM_SUM_RUN - 1) // NORM_SUM_RUN
    return max(cu_count(), runs) if m <= 16 else runs


def linear_fused(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
                 accumulate: bool = False, tiled: Optional[torch.Tensor] = None, swiglu: bool = False,
                 scale_in=None, norm_out=None) -> bool:
    """A bfloat16 product of at most 64 rows with an RMS norm folded in on either side, across two
    products: the norm is no kernel of its own between them (17 to 64 rows), and the product behind
    it reads its activations in bfloat16, half the bytes, with nothing to convert (at most 16 rows,
    where the norm is otherwise folded into that product's prologue):

    * `norm_out` = (g `[n]`, xg `[m][n]` bfloat16, sums `[m][norm_sum_parts(n, m)]`): the product stores
      or adds into the 32-bit `out` as `linear` does and leaves, beside it, bf16(out g) and the sums
      of out^2 in parts, for the norm with weight g that reads `out` next;
    * `scale_in` = (sums `[m][parts]`, eps): `x` is such an xg, and the product's sums are multiplied
      by the row's 1 / sqrt(sum / k + eps) before the bias and the epilogue; with `swiglu`, `weight`
      is `interleave_gate_up(Wg, Wu)` and out = silu(gate) * up, bfloat16.

    Returns False, having launched nothing, where the kernels the shape takes have no place for it
    (the caller then runs norm and product one after the other)."""
    _need(x, "linear_fused.x", torch.bfloat16)
    _need(weight, "linear_fused.weight", torch.bfloat16)
    m, k = x.shape
    n = weight.shape[0]
    if weight.shape[1] != k:
        raise KernelError(f"linear_fused: x is [{m},{k}], weight is {tuple(weight.shape)}")
    if m == 0 or m > 64 or (scale_in is None and norm_out is None):
        return False
    if swiglu:
        nf = out.shape[1]
        if n % 64 or not n // 2 - 32 < nf <= n // 2 or bias is not None or accumulate or norm_out is not None:
            raise KernelError(f"linear_fused(swiglu): weight {tuple(weight.shape)}, out {tuple(out.shape)}")
        _need(out, "linear_fused.out", torch.bfloat16, (m, nf))
        epi, ldc = EPI_SWIGLU, nf
    else:
        _need(out, "linear_fused.out", _FLOATS, (m, n))
        if accumulate and out.dtype != torch.float32:
            raise KernelError("linear_fused: accumulation needs a float32 output")
        epi = EPI_BF16 if out.dtype == torch.bfloat16 else (EPI_ACC_F32 if accumulate else EPI_F32)
        ldc = n
    if bias is not None:
        _need(bias, "linear_fused.bias", torch.float32, (n,))
    in_ssq, in_parts, in_eps = None, 0, 0.0
    if scale_in is not None:
        in_ssq, in_eps = scale_in
        _need(in_ssq, "linear_fused.scale_in", torch.float32)
        if in_ssq.dim() != 2 or in_ssq.shape[0] != m or in_ssq.shape[1] < 1:
            raise KernelError(f"linear_fused.scale_in: sums {tuple(in_ssq.shape)} for {m} rows")
        in_parts = in_ssq.shape[1]
    out_g = out_xg = out_ssq = None
    if norm_out is not None:
        out_g, out_xg, out_ssq = norm_out
        if out.dtype != torch.float32:
            raise KernelError("linear_fused.norm_out: the product's own output must be float32")
        _need(out_g, "linear_fused.norm_out.g", torch.float32, (n,))
        _need(out_xg, "linear_fused.norm_out.xg", torch.bfloat16, (m, n))
        _need(out_ssq, "linear_fused.norm_out.sums", torch.float32, (m, norm_sum_parts(n, m)))
    aligned = not (x.data_ptr() % 16 or weight.data_ptr() % 16 or k % 8)
    splits, per = _k_split(m, n, k, swiglu, aligned, tiled=tiled is not None)
    part = workspace("skinny", splits * m * n, x.device) if (splits > 1 or (swiglu and m > 16)) else None
    _need_tiled(tiled, "linear_fused.tiled", n, k)
    rc = _fn("gemm_bf16", "mf_gemm_bf16_skinny_fused")(
        _ptr(x), k, _ptr(weight), _ptr(tiled), k, _ptr(bias), _ptr(out), ldc, _ptr(part), m, n, k, splits, per, epi,
        _ptr(in_ssq), in_parts, float(in_eps), _ptr(out_g), _ptr(out_xg), _ptr(out_ssq),
        out_ssq.shape[1] if out_ssq is not None else 0, _stream())
    if rc == NOT_BUILT:
        return False
    _check(rc, f"gemm_bf16_skinny_fused{'(swiglu)' if swiglu else ''} {m}x{n}x{k}")
    return True


# ------------------------------------------------------------------ attention
def split_plan(n_tok: int, n_kv_heads: int, group: int, head_dim: int, max_len: int,
               target_blocks: int = 1024) -> Tuple[int, int]:
    """(n_splits, split_len) for the per-token attention: split the keys when tokens x kv
    heads alone do not fill the chip.  Depends on the capacity, not on current lengths;
    split_len is a multiple of the page size and at least four pages; at most 64 splits."""
    gc = 8 if head_dim <= 128 else 4
    blocks = n_tok * n_kv_heads * ((group + gc - 1) // gc)
    n_splits = max(1, min(target_blocks // max(1, blocks), (max_len + 4 * PAGE - 1) // (4 * PAGE), 64))
    split_len = ((max_len + n_splits - 1) // n_splits + PAGE - 1) // PAGE * PAGE
    return (max_len + split_len - 1) // split_len, split_len


def _need_caches(what: str, kcache: torch.Tensor, vcache: torch.Tensor, dtype, n_kv_heads: int,
                 head_dim: int) -> None:
    _need(kcache, what + ".kcache", dtype)
    _need(vcache, what + ".vcache", dtype)
    if tuple(kcache.shape[1:]) != (n_kv_heads, PAGE, head_dim):
        raise KernelError(f"{what}.kcache: shape {tuple(kcache.shape)}, expected "
                          f"[pages, {n_kv_heads}, {PAGE}, {head_dim}]")
    want = v_page_shape(n_kv_heads, head_dim, dtype)
    if tuple(vcache.shape[1:]) != want or vcache.shape[0] != kcache.shape[0]:
        raise KernelError(f"{what}.vcache: shape {tuple(vcache.shape)}, expected "
                          f"{[kcache.shape[0]] + list(want)}")


# Sequences that can be this long share their step's key splits by length: working the shares out
# costs a block about a microsecond, which shorter ones do not gain back.  (This threshold, the cap
# of four times the even share and the 32 places were tuned on an MI355X: 256 CUs in 8 dies.)
SHARED_SPLITS_FROM = 8192


def decode_split_plan(n_tok: int, n_kv_heads: int, group: int, max_len: int,
                      target_blocks: Optional[int] = None) -> Tuple[int, int]:
    """(places, splits) of the bfloat16 decode attention's key splits.  `splits`: about one block
    per CU, at least 256 keys of the longest possible sequence per split, at most 32.  A step of
    one token, of more than 64, of sequences that cannot be long, or without splits, gives every
    token that many (`places` = `splits`); otherwise the
    step's tokens share tokens x splits between them in proportion to their keys, a token taking
    at most `places` = 4 x splits (at most 32), so that a long sequence among short ones is cut
    finer and the blocks have about equal work.  The kernel divides a token's keys in rounds of
    128; a place without keys is marked empty and the merge passes it over."""
    if target_blocks is None:
        target_blocks = cu_count()
    blocks = n_tok * n_kv_heads * ((group + 15) // 16)
    splits = tuning.ATTN_SPLITS or max(1, min(target_blocks // max(1, blocks), (max_len + 255) // 256, 32))
    if n_tok == 1 or n_tok > 64 or splits == 1 or max_len < SHARED_SPLITS_FROM or tuning.ATTN_EQUAL_SPLITS:
        return splits, splits
    return max(splits, min(4 * splits, 32)), splits


def attn_tokens(q: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor, page_table: torch.Tensor,
                positions: torch.Tensor, seq_of_tok: torch.Tensor, out: torch.Tensor, n_heads: int,
                n_kv_heads: int, head_dim: int, scale: float, window: int, max_len: int) -> None:
    """Each query token attends to its sequence's cache rows lo..position.  `max_len` bounds
    position + 1 for every token (it only shapes the launch).  bfloat16 runs on the matrix
    cores, 32-bit on plain FMA."""
    n_tok = positions.numel()
    _need(q, "attn.q", _FLOATS, (n_tok, n_heads * head_dim))
    _need(out, "attn.out", q.dtype, (n_tok, n_heads * head_dim))
    _need_caches("attn", kcache, vcache, q.dtype, n_kv_heads, head_dim)
    _need(page_table, "attn.page_table", torch.int32)
    _need(positions, "attn.positions", torch.int32, (n_tok,))
    _need(seq_of_tok, "attn.seq_of_tok", torch.int32, (n_tok,))
    if head_dim % 16 or not 16 <= head_dim <= 256:
        raise KernelError(f"attention: head_dim {head_dim} is not a multiple of 16 in [16, 256]")
    if n_heads % n_kv_heads:
        raise KernelError(f"attention: {n_heads} heads are not a multiple of {n_kv_heads} kv heads")
    if max_len > page_table.shape[1] * PAGE:
        raise KernelError(f"attention: max_len {max_len} exceeds the page table ({page_table.shape[1]} pages)")
    if q.dtype == torch.bfloat16:
        n_splits, base = decode_split_plan(n_tok, n_kv_heads, n_heads // n_kv_heads, max_len)
        part = workspace("attn", n_tok * n_heads * n_splits * (head_dim + 2), q.device) if n_splits > 1 else None
        _check(_fn("attn_decode_bf16", "mf_attn_decode_bf16")(
            _ptr(q), _ptr(kcache), _ptr(vcache), _ptr(page_table), page_table.shape[1], _ptr(positions),
            _ptr(seq_of_tok), _ptr(out), _ptr(part), n_tok, n_heads, n_kv_heads, head_dim, float(scale),
            int(window or 0), n_splits, base, _stream()), "attn_decode_bf16")
        return
    n_splits, split_len = split_plan(n_tok, n_kv_heads, n_heads // n_kv_heads, head_dim, max_len)
    part = workspace("attn", n_tok * n_heads * n_splits * (head_dim + 2), q.device) if n_splits > 1 else None
    _check(_fn("attn_tokens_f32", "mf_attn_tokens_f32")(
        _ptr(q), _ptr(kcache), _ptr(vcache), _ptr(page_table), page_table.shape[1], _ptr(positions),
        _ptr(seq_of_tok), _ptr(out), _ptr(part), n_tok, n_heads, n_kv_heads, head_dim, float(scale),
        int(window or 0), n_splits, split_len, _stream()), "attn_tokens_f32")


def attn_decode_rope(qkv: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, kcache: torch.Tensor,
                     vcache: torch.Tensor, page_table: torch.Tensor, positions: torch.Tensor,
                     seq_of_tok: torch.Tensor, out: torch.Tensor, n_heads: int, n_kv_heads: int, head_dim: int,
                     scale: float, window: int, max_len: int, write_kv: bool = True) -> None:
    """A bfloat16 decode step's rotation, cache write and attention in one kernel: qkv is the
    float32 `[tokens][(heads + 2 kv_heads) head_dim]` output of the q|k|v product; every token is
    the next position of its sequence.  Same result as `rope_kvwrite` then `attn_tokens`."""
    n_tok = positions.numel()
    _need(qkv, "attn_decode_rope.qkv", torch.float32, (n_tok, (n_heads + 2 * n_kv_heads) * head_dim))
    _need(cos, "attn_decode_rope.cos", torch.float32)
    _need(sin, "attn_decode_rope.sin", torch.float32, tuple(cos.shape))
    if cos.shape[1] != head_dim // 2:
        raise KernelError(f"rope: table has {cos.shape[1]} frequencies, head_dim {head_dim} needs {head_dim // 2}")
    _need(out, "attn_decode_rope.out", torch.bfloat16, (n_tok, n_heads * head_dim))
    _need_caches("attn_decode_rope", kcache, vcache, torch.bfloat16, n_kv_heads, head_dim)
    _need(page_table, "attn_decode_rope.page_table", torch.int32)
    _need(positions, "attn_decode_rope.positions", torch.int32, (n_tok,))
    _need(seq_of_tok, "attn_decode_rope.seq_of_tok", torch.int32, (n_tok,))
    if head_dim % 16 or not 16 <= head_dim <= 256:
        raise KernelError(f"attention: head_dim {head_dim} is not a multiple of 16 in [16, 256]")
    if n_heads % n_kv_heads:
        raise KernelError(f"attention: {n_heads} heads are not a multiple of {n_kv_heads} kv heads")
    if max_len > page_table.shape[1] * PAGE or max_len > cos.shape[0]:
        raise KernelError(f"attention: max_len {max_len} exceeds the page table ({page_table.shape[1]} pages) "
                          f"or the rotation table ({cos.shape[0]} positions)")
    n_splits, base = decode_split_plan(n_tok, n_kv_heads, n_heads // n_kv_heads, max_len)
    part = workspace("attn", n_tok * n_heads * n_splits * (head_dim + 2), qkv.device) if n_splits > 1 else None
    _check(_fn("attn_decode_bf16", "mf_attn_decode_rope_bf16")(
        _ptr(qkv), _ptr(cos), _ptr(sin), _ptr(kcache), _ptr(vcache), _ptr(page_table), page_table.shape[1],
        _ptr(positions), _ptr(seq_of_tok), _ptr(out), _ptr(part), n_tok, n_heads, n_kv_heads, head_dim,
        float(scale), int(window or 0), n_splits, base, 1 if write_kv else 0, _stream()), "attn_decode_rope_bf16")


def prefill_tile(n_heads: int, n_kv_heads: int, head_dim: int):
    """(tq, gh, workgroups per block of queries): a workgroup of the prompt attention takes `gh` heads
    of a kv head's group (all of them, unless there are more than it has rows) times `tq` consecutive
    new tokens, so that a page of keys it brings in serves every head that reads it."""
    rows = _fn("attn_prefill_bf16", "mf_attn_prefill_rows")(head_dim)
    group = n_heads // n_kv_heads
    gh = min(group, rows)
    return rows // gh, gh, n_kv_heads * (-(-group // gh))


def attn_prefill(q: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor, page_table: torch.Tensor,
                 ctx, out: torch.Tensor, n_heads: int, n_kv_heads: int, head_dim: int, scale: float,
                 window: int) -> None:
    """bfloat16 attention of a step that brings several tokens per sequence: every new token
    attends to its sequence's cache rows up to its own position (the step's keys are already
    stored).  `ctx` gives the ragged layout (cu_seqlens, start_pos, the query blocks)."""
    n_tok = ctx.n_tokens
    _need(q, "attn_prefill.q", torch.bfloat16, (n_tok, n_heads * head_dim))
    _need(out, "attn_prefill.out", torch.bfloat16, (n_tok, n_heads * head_dim))
    _need_caches("attn_prefill", kcache, vcache, torch.bfloat16, n_kv_heads, head_dim)
    _need(page_table, "attn_prefill.page_table", torch.int32)
    if not scale > 0.0:
        raise KernelError(f"attn_prefill: scale {scale} must be positive")
    _need(ctx.cu_seqlens, "attn_prefill.cu_seqlens", torch.int32, (ctx.n_seqs + 1,))
    _need(ctx.start_pos, "attn_prefill.start_pos", torch.int32, (ctx.n_seqs,))
    if head_dim % 16 or not 16 <= head_dim <= 256:
        raise KernelError(f"attention: head_dim {head_dim} is not a multiple of 16 in [16, 256]")
    if n_heads % n_kv_heads:
        raise KernelError(f"attention: {n_heads} heads are not a multiple of {n_kv_heads} kv heads")
    if ctx.max_len > page_table.shape[1] * PAGE or page_table.shape[0] != ctx.n_seqs:
        raise KernelError(f"attention: page table {tuple(page_table.shape)} does not cover "
                          f"{ctx.n_seqs} sequences of up to {ctx.max_len} positions")
    # Where the kernel's time is that of the block with the most pages (a few new tokens on a long
    # context, few short prompts), blocks of queries with more pages than a workgroup's even share
    # of all of them (two workgroups fit a CU up to a head size of 128) are given to several
    # workgroups, which take the pages in turn.
    window = int(window or 0)
    tq, gh, per_tile = prefill_tile(n_heads, n_kv_heads, head_dim)
    per_cu = _fn("attn_prefill_bf16", "mf_attn_prefill_per_cu")(head_dim)
    shared = None if tuning.NO_SHARED_PAGES else ctx.shared_query_tiles(
        tq, PAGE, window, per_tile, cu_count(), per_cu, PREFILL_MIN_PAGES, PREFILL_MAX_SHARES)
    if shared is None:
        tile_seq, tile_q0 = ctx.query_tiles(tq)
        tile_share = parts = arrived = None
    else:
        tile_seq, tile_q0, tile_share, n_slots, most_shares = shared
        part = _fn("attn_prefill_bf16", "mf_attn_prefill_part_floats")(head_dim)
        parts = workspace("prefill_parts", n_slots * per_tile * most_shares * part, q.device)
        arrived = _zeroed_counters("prefill_arrived", n_slots * per_tile, q.device)
    rc = _fn("attn_prefill_bf16", "mf_attn_prefill_bf16")(
        _ptr(q), _ptr(kcache), _ptr(vcache), _ptr(page_table), page_table.shape[1], _ptr(ctx.cu_seqlens),
        _ptr(ctx.start_pos), _ptr(tile_seq), _ptr(tile_q0), _ptr(tile_share), _ptr(parts), _ptr(arrived),
        most_shares if shared is not None else 1, _ptr(out), tile_seq.numel(), n_heads, n_kv_heads, head_dim,
        gh, tq, float(scale), window, _stream())
    if rc != 0 and arrived is not None:
        arrived.zero_()                  # a launch that failed may have left workgroups counted in
    _check(rc, "attn_prefill_bf16")


# ------------------------------------------------------------------ sampling
def _logit_rows(logits: torch.Tensor, name: str):
    _need(logits, name, torch.float32)
    if logits.dim() != 2:
        raise KernelError(f"{name}: expected [rows][vocab], got {tuple(logits.shape)}")
    return logits.shape


def argmax(logits: torch.Tensor, out: torch.Tensor) -> None:
    rows, vocab = _logit_rows(logits, "argmax.logits")
    _need(out, "argmax.out", torch.int32, (rows,))
    chunks = 1
    if vocab >= 16384 and rows < 256:          # few long rows: several blocks per row
        chunks = max(1, min(64, 512 // rows, vocab // 4096))
    work = workspace("argmax", 2 * rows * chunks, logits.device) if chunks > 1 else None
    _check(_fn("sampling", "mf_argmax")(_ptr(logits), vocab, rows, vocab, _ptr(out), _ptr(work), chunks,
                                         _stream()), "argmax")


def sample(logits: torch.Tensor, temp: float, streams: torch.Tensor, steps: torch.Tensor,
           out: torch.Tensor, forced_r: Optional[torch.Tensor] = None) -> None:
    """Temperature draw per row (greedy when temp < 1e-6).  The uniform of row i is
    `rng.uniform(seed, key_i, steps[i])` for streams[i] = `rng.stream_i64(seed, key_i)`, or
    forced_r[i] when given (tests)."""
    rows, vocab = _logit_rows(logits, "sample.logits")
    _need(streams, "sample.streams", torch.int64, (rows,))
    _need(steps, "sample.steps", torch.int32, (rows,))
    _need(out, "sample.out", torch.int32, (rows,))
    if forced_r is not None:
        _need(forced_r, "sample.forced_r", torch.float32, (rows,))
    _check(_fn("sampling", "mf_sample")(_ptr(logits), vocab, rows, vocab, float(temp), _ptr(streams),
                                         _ptr(steps), _ptr(forced_r), _ptr(out), _stream()), "sample")


def penalties(logits: torch.Tensor, prev: torch.Tensor, n_prev: torch.Tensor, repeat: float,
              frequency: float, presence: float) -> None:
    rows, vocab = _logit_rows(logits, "penalties.logits")
    _need(prev, "penalties.prev", torch.int32)
    if prev.dim() != 2 or prev.shape[0] != rows:
        raise KernelError(f"penalties.prev: expected [{rows}][window], got {tuple(prev.shape)}")
    _need(n_prev, "penalties.n_prev", torch.int32, (rows,))
    _check(_fn("sampling", "mf_penalties")(_ptr(logits), vocab, rows, vocab, _ptr(prev), prev.shape[1],
                                            _ptr(n_prev), float(repeat), float(frequency),
                                            float(presence), _stream()), "penalties")


def top_k(logits: torch.Tensor, k: int) -> None:
    rows, vocab = _logit_rows(logits, "top_k.logits")
    _check(_fn("sampling", "mf_top_k")(_ptr(logits), vocab, rows, vocab, int(k), _stream()), "top_k")


def top_p(logits: torch.Tensor, p: float) -> None:
    rows, vocab = _logit_rows(logits, "top_p.logits")
    _check(_fn("sampling", "mf_top_p")(_ptr(logits), vocab, rows, vocab, float(p), _stream()), "top_p")


FILTERED_K_MAX = 48            # the largest top-k that `sample_filtered` takes
FILTERED_VOCAB_MAX = 64 * 64 * 64


def sample_filtered_takes(vocab: int, k: int, temp: float) -> bool:
    """Whether `sample_filtered` covers these settings (else: top_k, top_p, sample one after the other)."""
    return 1 <= k <= FILTERED_K_MAX and k < vocab <= FILTERED_VOCAB_MAX and temp >= 1e-6


def sample_filtered(logits: torch.Tensor, k: int, p: float, temp: float, streams: torch.Tensor,
                    steps: torch.Tensor, out: torch.Tensor, forced_r: Optional[torch.Tensor] = None) -> None:
    """top-k, then top-p (off unless 0 < p < 1), then the temperature draw, as `top_k`, `top_p` and
    `sample` one after the other give it, but reading each row once: its k largest entries and their
    ties are picked out by 64 waves a row and the rest runs on those few.  The logits stay as they
    are, except for rows with more equal values than the lists hold, which take the whole-row
    kernels in place."""
    rows, vocab = _logit_rows(logits, "sample_filtered.logits")
    if not sample_filtered_takes(vocab, k, temp):
        raise KernelError(f"sample_filtered: k {k}, vocabulary {vocab}, temperature {temp} are outside what it takes")
    _need(streams, "sample_filtered.streams", torch.int64, (rows,))
    _need(steps, "sample_filtered.steps", torch.int32, (rows,))
    _need(out, "sample_filtered.out", torch.int32, (rows,))
    if forced_r is not None:
        _need(forced_r, "sample_filtered.forced_r", torch.float32, (rows,))
    work = workspace("sample_filtered", rows * 64 * (2 * 64 + 2), logits.device)
    _check(_fn("sampling", "mf_sample_filtered")(_ptr(logits), vocab, rows, vocab, int(k), float(p), float(temp),
                                                  _ptr(streams), _ptr(steps), _ptr(forced_r), _ptr(work),
                                                  _ptr(out), _stream()),
           "sample_filtered")


def advance(next_ids: torch.Tensor, sampled: torch.Tensor, positions: torch.Tensor, steps: torch.Tensor,
            prev: Optional[torch.Tensor] = None, n_prev: Optional[torch.Tensor] = None,
            cursor: Optional[torch.Tensor] = None) -> None:
    """After a decode step: next_ids = sampled, positions and steps move on by one; with `prev`
    `[n][window]` the sampled token also enters the window of recent tokens (n_prev entries in
    use, cursor = where the next one goes)."""
    n = next_ids.numel()
    for name, t in (("next_ids", next_ids), ("sampled", sampled), ("positions", positions), ("steps", steps)):
        _need(t, "advance." + name, torch.int32, (n,))
    max_prev = 0
    if prev is not None:
        _need(prev, "advance.prev", torch.int32)
        if prev.dim() != 2 or prev.shape[0] != n:
            raise KernelError(f"advance.prev: shape {tuple(prev.shape)}, expected [{n}, window]")
        max_prev = prev.shape[1]
        _need(n_prev, "advance.n_prev", torch.int32, (n,))
        _need(cursor, "advance.cursor", torch.int32, (n,))
    _check(_fn("sampling", "mf_advance")(_ptr(next_ids), _ptr(sampled), _ptr(positions), _ptr(steps), n,
                                          _ptr(prev), max_prev, _ptr(n_prev if prev is not None else None),
                                          _ptr(cursor if prev is not None else None), _stream()), "advance")


# ------------------------------------------------------------------ measuring kernels
def probe_read(buffer: torch.Tensor, blocks: Optional[int] = None) -> None:
    """Launches one plain streaming read of the whole buffer (for the benchmark's measured
    memory bandwidth; time it from outside)."""
    _need(buffer, "probe_read.buffer")
    nbytes = buffer.numel() * buffer.element_size() // 16 * 16
    blocks = blocks or cu_count()
    sink = workspace("probe", blocks, buffer.device)
    _check(_fn("probe", "mf_probe_read")(_ptr(buffer), nbytes, _ptr(sink), blocks, _stream()), "probe_read")


def probe_mfma(rounds: int, blocks: Optional[int] = None, device="cuda") -> float:
    """Launches a register-resident loop of bfloat16 matrix-core products and returns the number
    of floating-point operations it performs (time it from outside)."""
    blocks = blocks or cu_count()
    sink = workspace("probe", blocks, device)
    _check(_fn("probe", "mf_probe_mfma")(int(rounds), _ptr(sink), blocks, _stream()), "probe_mfma")
    return float(blocks) * 8 * rounds * 8 * 2 * 32 * 32 * 16

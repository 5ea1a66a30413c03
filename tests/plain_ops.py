"""Plain torch versions of every HIP kernel, with the kernels' own signatures.

Two uses, both in tests only: (1) the reference each kernel is compared with on the GPU;
(2) patched over `minfer_amd.kernels.ops` (`install`), they let the CPU-only tests drive
the real engine, cache and generation loop where no GPU exists.  The product never imports
this file.  Arithmetic is float64 inside, rounded once to the output type.
"""
from __future__ import annotations

import math

import torch

PAGE = 64


def embed(table, ids, out):
    out.copy_(table[ids.long()].to(torch.float32))


def rmsnorm(x, weight, eps, out, row_idx=None):
    src = x if row_idx is None else x[row_idx.long()]
    s = src.double()
    y = s * (1.0 / torch.sqrt((s * s).mean(dim=-1, keepdim=True) + eps))
    if weight is not None:
        y = y * weight.double()
    out.copy_(y.to(out.dtype))


def rmsnorm_reference(x, weight, eps):
    """The norm alone, float64, unrounded."""
    s = x.double()
    return s * (1.0 / torch.sqrt((s * s).mean(dim=-1, keepdim=True) + eps)) * weight.double()


def gather_rows(x, idx, out):
    out.copy_(x[idx.long()])


def swiglu(gate_up, out):
    nf = gate_up.shape[1] // 2
    g, u = gate_up[:, :nf].double(), gate_up[:, nf:].double()
    out.copy_((g / (1.0 + torch.exp(-g)) * u).to(out.dtype))


def convert(src, dst):
    dst.copy_(src.to(dst.dtype))


def fill_normal(out, seed, std, round_bf16=True):
    """The library's own host fill: the numbers are defined by csrc/random_normal.h, on both sides."""
    from minfer_amd.kernels import ops
    ops.fill_normal_host(out, seed, std, round_bf16)


def rope_table(n_pos, half, theta, freq_scale, device):
    i = torch.arange(half, dtype=torch.float64)
    freq = freq_scale / torch.pow(torch.tensor(float(theta), dtype=torch.float64), 2.0 * i / (2 * half))
    ang = torch.arange(n_pos, dtype=torch.float64)[:, None] * freq[None, :]
    return torch.cos(ang).float().to(device), torch.sin(ang).float().to(device)


def rope_kvwrite(qkv, cos, sin, positions, seq_of_tok, page_table, q_out, kcache, vcache,
                 n_heads, n_kv_heads, head_dim, write_kv=True):
    t = positions.numel()
    half = head_dim // 2
    x = qkv.double().view(t, n_heads + 2 * n_kv_heads, head_dim)
    if cos is None:                      # nothing is rotated: q is rounded, k and v are stored
        c, s = torch.ones(t, 1, half, dtype=torch.float64), torch.zeros(t, 1, half, dtype=torch.float64)
    else:
        c = cos[positions.long()].double()[:, None, :]
        s = sin[positions.long()].double()[:, None, :]

    def rot(v):
        v0, v1 = v[..., :half], v[..., half:]
        return torch.cat([v0 * c - v1 * s, v0 * s + v1 * c], dim=-1)
    q_out.copy_(rot(x[:, :n_heads]).reshape(t, n_heads * head_dim).to(q_out.dtype))
    if not write_kv:
        return
    k = rot(x[:, n_heads:n_heads + n_kv_heads]).to(kcache.dtype)
    v = x[:, n_heads + n_kv_heads:].to(vcache.dtype)
    pos = positions.long()
    page = page_table.long()[seq_of_tok.long(), pos // PAGE]
    assert (page >= 0).all(), "token written to a page that was not reserved"
    kcache[page, :, pos % PAGE, :] = k
    if v_transposed(vcache):
        vcache[page, :, (pos % PAGE) // 32, :, pos % 32] = v
    else:
        vcache[page, :, pos % PAGE, :] = v


def rope_inplace(qkv, cos, sin, positions, n_rot_heads, n_heads_total, head_dim):
    t, half = positions.numel(), head_dim // 2
    x = qkv.view(t, n_heads_total, head_dim)
    c = cos[positions.long()].double()[:, None, :]
    s = sin[positions.long()].double()[:, None, :]
    v = x[:, :n_rot_heads].double()
    v0, v1 = v[..., :half], v[..., half:]
    x[:, :n_rot_heads] = torch.cat([v0 * c - v1 * s, v0 * s + v1 * c], dim=-1).float()


def linear(x, weight, bias, out, accumulate=False, variant=0, tiled=None):
    y = x.double() @ weight.double().t()
    if bias is not None:
        y = y + bias.double()
    if accumulate:
        y = y + out.double()
    out.copy_(y.to(out.dtype))


def interleave_gate_up(gate, up):
    """The layout the fused kernel reads, built row by row."""
    nf, k = gate.shape
    groups = (nf + 31) // 32
    out = torch.zeros(groups * 64, k, dtype=gate.dtype)
    for i in range(nf):
        out[(i // 32) * 64 + i % 32] = gate[i]
        out[(i // 32) * 64 + 32 + i % 32] = up[i]
    return out


def linear_swiglu(x, weight, out, variant=0, tiled=None):
    nf = out.shape[1]
    idx = torch.arange(nf)
    g = x.double() @ weight.double()[(idx // 32) * 64 + idx % 32].t()
    u = x.double() @ weight.double()[(idx // 32) * 64 + 32 + idx % 32].t()
    out.copy_((g / (1.0 + torch.exp(-g)) * u).to(out.dtype))


def linear_normed(x, norm_weight, eps, row_idx, weight, bias, out, accumulate=False, swiglu=False, tiled=None):
    """The stand-in has no folded kernel: the caller norms and multiplies in two steps."""
    return False


def linear_fused(x, weight, bias, out, accumulate=False, tiled=None, swiglu=False, scale_in=None, norm_out=None):
    """The stand-in folds no norm around a product: the caller runs the norm as a step of its own."""
    return False


def linear_normed_reference(x, norm_weight, eps, row_idx, weight, bias, swiglu=False):
    """What the folded kernel computes, in float64, with its one rounding of the activations:
    bf16(x * g) goes to the matrix cores and 1 / sqrt(mean(x^2) + eps) is applied to the sums."""
    rows = x if row_idx is None else x[row_idx.long()]
    a = (rows.float() * norm_weight.float()).to(torch.bfloat16).double()
    inv = 1.0 / torch.sqrt((rows.double() ** 2).mean(dim=1, keepdim=True) + eps)
    y = a @ weight.double().t() * inv
    if bias is not None:
        y = y + bias.double()
    return y


def v_transposed(vcache):
    """A bfloat16 cache keeps a page of V as [kv_heads][2][head_dim][32] (key j is element j % 32
    of half j / 32), a 32-bit one as [kv_heads][64][head_dim] (the product's `v_page_shape`)."""
    return vcache.dtype == torch.bfloat16


def v_rows(vcache, page, off):
    """[n][kv_heads][head_dim] rows of V at (page[i], off[i])."""
    return vcache[page, :, off // 32, :, off % 32] if v_transposed(vcache) else vcache[page, :, off, :]


def gather_cache_rows(cache, page_table_row, length, is_v=False):
    """[length][kv_heads][head_dim] rows 0..length-1 of one sequence."""
    pos = torch.arange(length)
    page = page_table_row.long()[pos // PAGE]
    return v_rows(cache, page, pos % PAGE) if is_v else cache[page, :, pos % PAGE, :]


def attn_tokens(q, kcache, vcache, page_table, positions, seq_of_tok, out, n_heads, n_kv_heads,
                head_dim, scale, window, max_len):
    t = positions.numel()
    g = n_heads // n_kv_heads
    qh = q.double().view(t, n_heads, head_dim)
    res = torch.zeros(t, n_heads, head_dim, dtype=torch.float64)
    for i in range(t):
        p = int(positions[i])
        lo = max(0, p - window + 1) if window else 0
        row = page_table[int(seq_of_tok[i])]
        pos = torch.arange(lo, p + 1)
        page = row.long()[pos // PAGE]
        assert (page >= 0).all(), "attention reads a page that was given back"
        k = kcache[page, :, pos % PAGE, :].double()      # [n][nk][hd]
        v = v_rows(vcache, page, pos % PAGE).double()
        for h in range(n_heads):
            s = (k[:, h // g, :] @ qh[i, h]) * scale
            res[i, h] = torch.softmax(s, dim=0) @ v[:, h // g, :]
    out.copy_(res.view(t, n_heads * head_dim).to(out.dtype))


def attn_decode_rope(qkv, cos, sin, kcache, vcache, page_table, positions, seq_of_tok, out, n_heads,
                     n_kv_heads, head_dim, scale, window, max_len, write_kv=True):
    q = torch.empty(positions.numel(), n_heads * head_dim, dtype=out.dtype)
    rope_kvwrite(qkv, cos, sin, positions, seq_of_tok, page_table, q, kcache, vcache, n_heads, n_kv_heads,
                 head_dim, write_kv)
    attn_tokens(q, kcache, vcache, page_table, positions, seq_of_tok, out, n_heads, n_kv_heads, head_dim, scale,
                window, max_len)


def attn_prefill(q, kcache, vcache, page_table, ctx, out, n_heads, n_kv_heads, head_dim, scale, window):
    attn_tokens(q, kcache, vcache, page_table, ctx.positions, ctx.seq_of_tok, out, n_heads, n_kv_heads,
                head_dim, scale, window, ctx.max_len)


# ------------------------------------------------------------------ sampling
def argmax(logits, out):
    import plain_qwen2 as pq
    for i in range(logits.shape[0]):
        out[i] = pq.greedy(logits[i].numpy())


def stream_uniform(stream_i64: int, step: int) -> float:
    """The draw of a stream id (as an int64 tensor holds it) at a step: the device's uniform01."""
    from minfer_amd.sampling.rng import mix64
    h = mix64((stream_i64 & 0xFFFFFFFFFFFFFFFF) ^ (step & 0xFFFFFFFFFFFFFFFF))
    return (h >> 40) / 16777216.0


def sample(logits, temp, streams, steps, out, forced_r=None):
    import plain_qwen2 as pq
    for i in range(logits.shape[0]):
        if temp < 1e-6:
            out[i] = pq.greedy(logits[i].numpy())
            continue
        r = float(forced_r[i]) if forced_r is not None else stream_uniform(int(streams[i]), int(steps[i]))
        out[i] = pq.sample_from_probs(pq.temperature_probs(logits[i].numpy(), temp), r)


def penalties(logits, prev, n_prev, repeat, frequency, presence):
    import plain_qwen2 as pq
    for i in range(logits.shape[0]):
        window = prev[i, :int(n_prev[i])].tolist()
        logits[i] = torch.from_numpy(pq.apply_penalties(logits[i].numpy(), window, repeat, frequency, presence))


def top_k(logits, k):
    import plain_qwen2 as pq
    for i in range(logits.shape[0]):
        logits[i] = torch.from_numpy(pq.apply_top_k(logits[i].numpy(), k))


def top_p(logits, p):
    import plain_qwen2 as pq
    for i in range(logits.shape[0]):
        logits[i] = torch.from_numpy(pq.apply_top_p(logits[i].numpy(), p))


def sample_filtered_takes(vocab, k, temp):
    return 1 <= k <= 48 and k < vocab <= 32 * 256 * 32 and temp >= 1e-6


def sample_filtered(logits, k, p, temp, streams, steps, out, forced_r=None):
    work = logits.clone()
    top_k(work, k)
    if 0.0 < p < 1.0:
        top_p(work, p)
    sample(work, temp, streams, steps, out, forced_r)


def advance(next_ids, sampled, positions, steps, prev=None, n_prev=None, cursor=None):
    next_ids.copy_(sampled)
    positions += 1
    steps += 1
    if prev is not None:
        for i in range(next_ids.numel()):
            c = int(cursor[i])
            prev[i, c] = sampled[i]
            cursor[i] = (c + 1) % prev.shape[1]
            n_prev[i] = min(int(n_prev[i]) + 1, prev.shape[1])


NAMES = ["embed", "rmsnorm", "gather_rows", "swiglu", "convert", "fill_normal", "rope_table",
         "rope_kvwrite", "rope_inplace", "linear", "attn_tokens", "attn_prefill", "argmax", "sample", "penalties",
         "top_k", "top_p", "sample_filtered", "sample_filtered_takes", "advance", "interleave_gate_up", "linear_swiglu", "linear_normed", "linear_fused", "attn_decode_rope"]


def install(monkeypatch):
    """Replaces the HIP launchers by the plain versions and lets models live on the CPU."""
    from minfer_amd.engine import loading
    from minfer_amd.kernels import ops
    for name in NAMES:
        monkeypatch.setattr(ops, name, globals()[name], raising=False)
    monkeypatch.setattr(loading, "require_gpu", lambda device: torch.device("cpu"))

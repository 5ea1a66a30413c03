"""Each HIP kernel alone against its plain torch version (tests/plain_ops.py), at sizes
other than the engine's: widths and vocabularies that are no power of two, partial tiles,
head sizes in steps of 16, several group sizes."""
import math

import numpy as np
import pytest
import torch

import plain_ops

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    from minfer_amd.kernels import ops as o
    return o


def rnd(shape, dtype=torch.float32, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


def close(a, b, atol, rtol=0.0):
    a, b = a.detach().cpu().double(), b.detach().cpu().double()
    err = (a - b).abs()
    lim = atol + rtol * b.abs()
    assert bool((err <= lim).all()), f"max err {err.max().item():.3e} (limit {atol}+{rtol}*|ref|)"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,d,vocab", [(1, 64, 50), (7, 200, 777), (33, 3584, 1000)])
def test_embed(ops, dtype, rows, d, vocab):
    table = rnd((vocab, d), dtype, 1)
    ids = torch.randint(0, vocab, (rows,), dtype=torch.int32)
    out = torch.empty(rows, d, dtype=torch.float32, device=DEV)
    ops.embed(table.to(DEV), ids.to(DEV), out)
    ref = torch.empty(rows, d)
    plain_ops.embed(table, ids, ref)
    assert torch.equal(out.cpu(), ref)


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,d,eps", [(1, 64, 1e-6), (5, 200, 1e-5), (130, 3584, 1e-6), (3, 1000, 0.1),
                                         (2, 5120, 1e-5), (3, 8192, 1e-5), (2, 12288, 1e-6), (2, 20000, 1e-6),
                                         (2, 4099, 1e-6)])
def test_rmsnorm(ops, out_dtype, rows, d, eps):
    x = rnd((rows, d), seed=2, scale=3.0)
    w = rnd((d,), seed=3) + 1.0
    out = torch.empty(rows, d, dtype=out_dtype, device=DEV)
    ops.rmsnorm(x.to(DEV), w.to(DEV), eps, out)
    ref = torch.empty(rows, d, dtype=torch.float64)
    plain_ops.rmsnorm(x, w, eps, ref)
    tol = 2e-6 if out_dtype == torch.float32 else 1e-2
    close(out, ref, tol * 3, tol)
    # with a row gather
    idx = torch.tensor([rows - 1, 0, rows // 2], dtype=torch.int32)
    out2 = torch.empty(3, d, dtype=out_dtype, device=DEV)
    ops.rmsnorm(x.to(DEV), w.to(DEV), eps, out2, idx.to(DEV))
    close(out2, ref[idx.long()], tol * 3, tol)


def test_gather_rows(ops):
    x = torch.tensor([[1., 2, 3, 4], [10, 20, 30, 40], [100, 200, 300, 400]])
    idx = torch.tensor([2, 0], dtype=torch.int32)
    out = torch.empty(2, 4, device=DEV)
    ops.gather_rows(x.to(DEV), idx.to(DEV), out)
    assert out.cpu().tolist() == [[100, 200, 300, 400], [1, 2, 3, 4]]


@pytest.mark.parametrize("in_dtype,out_dtype", [(torch.float32, torch.float32), (torch.float32, torch.bfloat16),
                                                (torch.bfloat16, torch.bfloat16)])
@pytest.mark.parametrize("rows,nf", [(1, 176), (9, 344), (64, 18944)])
def test_swiglu(ops, in_dtype, out_dtype, rows, nf):
    gu = rnd((rows, 2 * nf), in_dtype, 4, 3.0)
    gu[0, :4] = torch.tensor([0.0, 88.0, -88.0, 30.0]).to(in_dtype)
    out = torch.empty(rows, nf, dtype=out_dtype, device=DEV)
    ops.swiglu(gu.to(DEV), out)
    ref = torch.empty(rows, nf, dtype=torch.float64)
    plain_ops.swiglu(gu, ref)
    assert torch.isfinite(out).all()
    tol = 1e-6 if out_dtype == torch.float32 else 8e-3
    close(out, ref, tol, tol)


def test_convert(ops):
    x = rnd((1000, 37), seed=5)
    b = torch.empty(1000, 37, dtype=torch.bfloat16, device=DEV)
    ops.convert(x.to(DEV), b)
    assert torch.equal(b.cpu(), x.to(torch.bfloat16))
    f = torch.empty(1000, 37, dtype=torch.float32, device=DEV)
    ops.convert(b, f)
    assert torch.equal(f.cpu(), x.to(torch.bfloat16).float())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_fill_normal(ops, dtype):
    a = torch.empty(1 << 20, dtype=dtype, device=DEV)
    b = torch.empty(1 << 20, dtype=dtype, device=DEV)
    ops.fill_normal(a, 1234, 0.02)
    ops.fill_normal(b, 1234, 0.02)
    assert torch.equal(a, b)
    ops.fill_normal(b, 1235, 0.02)
    assert not torch.equal(a, b)
    a = a.float().cpu()
    assert abs(a.mean().item()) < 2e-4 and abs(a.std().item() - 0.02) < 2e-4
    assert a.abs().max().item() < 0.02 * 7


@pytest.mark.parametrize("theta,half", [(10000.0, 8), (1e6, 64), (50000.0, 24)])
def test_rope_table(ops, theta, half):
    cs, sn = ops.rope_table(300, half, theta, 1.0, DEV)
    rc, rs = plain_ops.rope_table(300, half, theta, 1.0, "cpu")
    close(cs, rc, 2e-7)
    close(sn, rs, 2e-7)


def test_rope_table_frequency_ladder_by_hand(ops):
    """freq_i = theta^(-2i/hd): with head_dim 8 and theta 10^4 the frequencies are 1, 0.1, 0.01
    and 0.001, so row 1000 of the table holds cos and sin of 1000, 100, 10 and 1 radians (values
    from tables, not from the formula; src/graph/cpu_backend.rs:415 of yusiwen/minfer)."""
    cs, sn = ops.rope_table(1001, 4, 10000.0, 1.0, DEV)
    want_c = [0.5623790762907029, 0.8623188722876839, -0.8390715290764524, 0.5403023058681398]
    want_s = [0.8268795405320025, -0.5063656411097588, -0.5440211108893698, 0.8414709848078965]
    assert (cs[1000].double().cpu() - torch.tensor(want_c, dtype=torch.float64)).abs().max() < 1e-6
    assert (sn[1000].double().cpu() - torch.tensor(want_s, dtype=torch.float64)).abs().max() < 1e-6
    assert abs(cs[1, 0].item() - 0.5403023058681398) < 1e-7 and abs(sn[1, 0].item() - 0.8414709848078965) < 1e-7


def make_cache(n_pages, nk, hd, dtype, seed=0):
    """K and V as [pages][kv_heads][64][head_dim]: for V this is the logical view, `stored_v`
    gives what the kernels take."""
    k = rnd((n_pages, nk, 64, hd), dtype, seed)
    v = rnd((n_pages, nk, 64, hd), dtype, seed + 1)
    return k, v


def stored_v(v):
    """A bfloat16 cache keeps a page of V transposed in two halves, [kv_heads][2][head_dim][32]."""
    if v.dtype != torch.bfloat16:
        return v
    pages, nk, _, hd = v.shape
    return v.view(pages, nk, 2, 32, hd).transpose(3, 4).contiguous()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,nk,hd", [(4, 2, 16), (9, 3, 48), (28, 4, 128), (2, 2, 256)])
def test_rope_kvwrite(ops, dtype, nh, nk, hd):
    # three sequences with scattered pages; tokens at positions straddling a page edge
    pos = torch.tensor([0, 1, 62, 63, 64, 65, 5, 130], dtype=torch.int32)
    seq = torch.tensor([0, 0, 1, 1, 1, 1, 2, 2], dtype=torch.int32)
    table = torch.tensor([[5, -1, -1], [7, 2, -1], [0, 3, 9]], dtype=torch.int32)
    t = pos.numel()
    qkv = rnd((t, (nh + 2 * nk) * hd), seed=6)
    cs, sn = plain_ops.rope_table(256, hd // 2, 1e4, 1.0, "cpu")
    kc, vc = make_cache(10, nk, hd, dtype, 7)
    vc = stored_v(vc)
    q_ref = torch.empty(t, nh * hd, dtype=dtype)
    kr, vr = kc.clone(), vc.clone()
    plain_ops.rope_kvwrite(qkv, cs, sn, pos, seq, table, q_ref, kr, vr, nh, nk, hd)
    q = torch.empty(t, nh * hd, dtype=dtype, device=DEV)
    kd, vd = kc.to(DEV), vc.to(DEV)
    ops.rope_kvwrite(qkv.to(DEV), cs.to(DEV), sn.to(DEV), pos.to(DEV), seq.to(DEV), table.to(DEV), q,
                     kd, vd, nh, nk, hd)
    tol = 2e-6 if dtype == torch.float32 else 2e-2
    close(q, q_ref, tol, tol)
    close(kd, kr, tol, tol)
    close(vd, vr, tol, tol)
    # untouched rows stay untouched
    assert torch.equal(kd.cpu()[1], kc[1]) and torch.equal(vd.cpu()[4], vc[4])
    # the same from a q|k|v buffer that starts 4 bytes off a 16-byte boundary: the kernel
    # without 16-byte loads, same result up to how the compiler fuses the multiply-adds
    flat = torch.empty(qkv.numel() + 1, device=DEV)
    odd = flat[1:].view(qkv.shape)
    odd.copy_(qkv)
    assert odd.data_ptr() % 16 == 4 and odd.is_contiguous()
    q2 = torch.empty(t, nh * hd, dtype=dtype, device=DEV)
    kd2, vd2 = kc.to(DEV), vc.to(DEV)
    ops.rope_kvwrite(odd, cs.to(DEV), sn.to(DEV), pos.to(DEV), seq.to(DEV), table.to(DEV), q2, kd2, vd2, nh, nk, hd)
    close(q2, q_ref, tol, tol)
    close(kd2, kr, tol, tol)
    close(vd2, vr, tol, tol)


def test_rope_position_zero_is_identity_and_pairs_are_half_split(ops):
    nh, nk, hd = 2, 1, 32
    qkv = torch.zeros(2, (nh + 2 * nk) * hd)
    qkv[:, 3] = 1.0                      # element 3 of head 0
    cs, sn = ops.rope_table(64, hd // 2, 100.0, 1.0, DEV)
    pos = torch.tensor([0, 9], dtype=torch.int32, device=DEV)
    seq = torch.zeros(2, dtype=torch.int32, device=DEV)
    table = torch.zeros(1, 1, dtype=torch.int32, device=DEV)
    kc = torch.zeros(1, nk, 64, hd, device=DEV)
    vc = torch.zeros(1, nk, 64, hd, device=DEV)
    q = torch.empty(2, nh * hd, device=DEV)
    ops.rope_kvwrite(qkv.to(DEV), cs, sn, pos, seq, table, q, kc, vc, nh, nk, hd)
    q = q.cpu()
    assert torch.equal(q[0], qkv[0, :nh * hd])
    nz = torch.nonzero(q[1]).flatten().tolist()
    assert nz == [3, 3 + hd // 2]        # energy moves to i + hd/2, not to i + 1
    ang = 9.0 / 100.0 ** (2 * 3 / hd)
    assert abs(q[1, 3].item() - math.cos(ang)) < 1e-6 and abs(q[1, 3 + hd // 2].item() - math.sin(ang)) < 1e-6


GEMM_SHAPES = [(1, 64, 64), (3, 176, 64), (17, 1000, 344), (64, 512, 128), (65, 200, 232), (130, 777, 200),
               (300, 4608, 3584), (33, 96, 18944)]


@pytest.mark.parametrize("m,n,k", GEMM_SHAPES)
def test_gemm_f32(ops, m, n, k):
    x, w, b = rnd((m, k), seed=8), rnd((n, k), seed=9, scale=0.05), rnd((n,), seed=10)
    ref = x.double() @ w.double().t() + b.double()
    out = torch.empty(m, n, device=DEV)
    ops.linear(x.to(DEV), w.to(DEV), b.to(DEV), out)
    close(out, ref, 1e-5 * math.sqrt(k) / 8, 1e-5)
    base = rnd((m, n), seed=11)
    acc = base.to(DEV).clone()
    ops.linear(x.to(DEV), w.to(DEV), None, acc, accumulate=True)
    close(acc, ref - b.double() + base.double(), 1e-5 * math.sqrt(k) / 8, 1e-5)


@pytest.mark.parametrize("variant", [0, 1, 2, 3, 6, 9, 12, 13, 15])
@pytest.mark.parametrize("m,n,k", GEMM_SHAPES + [(2048, 512, 256), (1, 152064, 64), (64, 3584, 3584),
                                                 # at most 16 rows with K of 1536..4096: activations in registers
                                                 (1, 2100, 1536), (5, 2050, 2048), (8, 4001, 3584), (16, 2048, 4096),
                                                 # K of 5120 and 8192: the weights go through a shorter ring
                                                 (5, 2100, 5120), (8, 4100, 5120), (3, 5000, 8192), (16, 8192, 8192),
                                                 # 17..64 rows, whole chunks of K: the ring kernel, with K split
                                                 (20, 200, 768), (50, 1000, 4096),
                                                 # 9..16 rows against a long K: the same kernel
                                                 (12, 300, 8192), (16, 3584, 18944), (4, 5120, 8192),
                                                 # more than 64 rows but few tiles: K split over blocks
                                                 (200, 3584, 18944), (65, 1000, 1100), (512, 777, 2048),
                                                 # many rows, few big tiles, a long K: K split over 256 x 256 tiles
                                                 (800, 300, 4096), (1030, 777, 6144),
                                                 # tiles of 256 x 192 and 256 x 128 where the 256-wide ones leave CUs idle
                                                 (2048, 4608, 512), (1100, 3584, 1024), (8192, 1000, 192)])
def test_gemm_bf16(ops, variant, m, n, k):
    if variant and (m * n * k > 3e9):
        pytest.skip("large shape is covered by the default variant")
    if variant >= 12 and k % 64:
        pytest.skip("the direct-to-LDS kernel takes K in multiples of 64")
    x, w, b = rnd((m, k), torch.bfloat16, 8), rnd((n, k), torch.bfloat16, 9, 0.05), rnd((n,), seed=10)
    ref = x.double() @ w.double().t() + b.double()
    xd, wd, bd = x.to(DEV), w.to(DEV), b.to(DEV)
    tol = 2e-5 * math.sqrt(k)
    out = torch.empty(m, n, device=DEV)
    ops.linear(xd, wd, bd, out, variant=variant)
    close(out, ref, tol, 1e-5)
    out2 = torch.empty(m, n, device=DEV)
    ops.linear(xd, wd, bd, out2, variant=variant)
    assert torch.equal(out, out2), "two runs differ"
    base = rnd((m, n), seed=11)
    acc = base.to(DEV).clone()
    ops.linear(xd, wd, None, acc, accumulate=True, variant=variant)
    close(acc, ref - b.double() + base.double(), tol, 1e-5)
    ob = torch.empty(m, n, dtype=torch.bfloat16, device=DEV)
    ops.linear(xd, wd, bd, ob, variant=variant)
    close(ob, ref, tol, 8e-3)


def test_gemm_reference_vector(ops):
    # src/graph/cpu_backend.rs:540-566: W diag-like, b, x -> then silu and *2
    w = torch.tensor([[1., 0, 0, 0], [0, 2, 0, 0], [0, 0, 3, 0]])
    b = torch.tensor([0.5, -1.0, 0.25])
    x = torch.tensor([[1., 2, 3, 4]])
    out = torch.empty(1, 3, device=DEV)
    ops.linear(x.to(DEV), w.to(DEV), b.to(DEV), out)
    assert out.cpu().tolist() == [[1.5, 3.0, 9.25]]
    ob = torch.empty(1, 3, device=DEV)
    ops.linear(x.to(DEV).bfloat16(), w.to(DEV).bfloat16(), b.to(DEV), ob)
    assert ob.cpu().tolist() == [[1.5, 3.0, 9.25]]


def poison_unwritten(kc, vc, table, lengths):
    """Rows of a page after its sequence's last token were never written: a page is not
    cleared when it is taken, so they may hold anything.  NaN makes a kernel that touches
    them show."""
    for b, l in enumerate(lengths):
        if l % 64:
            page = int(table[b, l // 64])
            kc[page, :, l % 64:] = float("nan")
            vc[page, :, l % 64:] = float("nan")


def build_attention_case(nh, nk, hd, lengths, dtype, seed, n_pages_extra=3):
    """Sequences of the given lengths in shuffled pages; one query token per sequence at its
    last position, plus a few mid-sequence queries."""
    rng = np.random.default_rng(seed)
    n_cols = max((l + 63) // 64 for l in lengths)
    n_pages = sum((l + 63) // 64 for l in lengths) + n_pages_extra
    perm = rng.permutation(n_pages)
    table = -np.ones((len(lengths), n_cols), dtype=np.int32)
    nxt = 0
    for b, l in enumerate(lengths):
        for c in range((l + 63) // 64):
            table[b, c] = perm[nxt]
            nxt += 1
    kc, vc = make_cache(n_pages, nk, hd, dtype, seed)
    poison_unwritten(kc, vc, table, lengths)
    pos, seq = [], []
    for b, l in enumerate(lengths):
        for p in sorted({l - 1, l // 2, 0}):
            pos.append(p)
            seq.append(b)
    pos = torch.tensor(pos, dtype=torch.int32)
    seq = torch.tensor(seq, dtype=torch.int32)
    q = rnd((pos.numel(), nh * hd), dtype, seed + 5)
    return q, kc, stored_v(vc), torch.from_numpy(table), pos, seq


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,nk,hd,window", [(4, 2, 16, 0), (4, 1, 32, 0), (9, 3, 48, 0), (28, 4, 128, 0),
                                             (8, 8, 64, 0), (20, 2, 80, 0), (4, 2, 256, 0), (4, 2, 64, 40),
                                             (12, 1, 128, 100)])
def test_attn_tokens(ops, dtype, nh, nk, hd, window):
    lengths = [1, 5, 30, 33, 64, 65, 100, 240, 1000]
    q, kc, vc, table, pos, seq = build_attention_case(nh, nk, hd, lengths, dtype, 12)
    scale = 1.0 / math.sqrt(hd)
    ref = torch.empty(q.shape, dtype=torch.float64)
    plain_ops.attn_tokens(q, kc, vc, table, pos, seq, ref, nh, nk, hd, scale, window, max(lengths))
    dq, dk, dv, dt, dp, ds = (t.to(DEV) for t in (q, kc, vc, table, pos, seq))
    tol = 3e-6 if dtype == torch.float32 else 1.5e-2
    outs = []
    for max_len in (max(lengths), 4096):          # different key splits, same result
        out = torch.empty(q.shape, dtype=dtype, device=DEV)
        ops.attn_tokens(dq, dk, dv, dt if max_len <= table.shape[1] * 64 else
                        torch.nn.functional.pad(dt, (0, 64 - table.shape[1]), value=-1).contiguous(),
                        dp, ds, out, nh, nk, hd, scale, window, max_len)
        close(out, ref, tol, tol)
        outs.append(out)
    again = torch.empty(q.shape, dtype=dtype, device=DEV)
    ops.attn_tokens(dq, dk, dv, dt, dp, ds, again, nh, nk, hd, scale, window, max(lengths))
    assert torch.equal(again, outs[0]), "two runs differ"


@pytest.mark.parametrize("write_kv", [True, False])
@pytest.mark.parametrize("nh,nk,hd,window", [(4, 2, 16, 0), (9, 3, 48, 0), (28, 4, 128, 0), (20, 1, 80, 0),
                                             (4, 2, 256, 0), (4, 2, 64, 40), (36, 2, 128, 0)])
def test_attn_decode_rope(ops, nh, nk, hd, window, write_kv):
    """Rotation + cache write + attention of a decode step in one kernel against the two-step
    plain path.  The row of the token's own position is poisoned beforehand when the kernel
    is to write it: it must take k and v from the product's output, not from the cache."""
    decode_rope_case(ops, nh, nk, hd, window, write_kv, [1, 2, 31, 32, 33, 64, 65, 129, 500, 1000])


def decode_rope_case(ops, nh, nk, hd, window, write_kv, lengths):
    rng = np.random.default_rng(31)
    n_cols = max((l + 63) // 64 for l in lengths)
    n_pages = sum((l + 63) // 64 for l in lengths) + 3
    perm = rng.permutation(n_pages)
    table = -np.ones((len(lengths), n_cols), dtype=np.int32)
    nxt = 0
    for b, l in enumerate(lengths):
        for c in range((l + 63) // 64):
            table[b, c] = perm[nxt]
            nxt += 1
    kc, vc = make_cache(n_pages, nk, hd, torch.bfloat16, 32)
    # rows from the token's own position on are unwritten; with write_kv False the own row exists
    poison_unwritten(kc, vc, table, [l - 1 if write_kv else l for l in lengths])
    vc = stored_v(vc)
    table = torch.from_numpy(table)
    pos = torch.tensor([l - 1 for l in lengths], dtype=torch.int32)
    seq = torch.arange(len(lengths), dtype=torch.int32)
    qkv = rnd((len(lengths), (nh + 2 * nk) * hd), seed=33)
    longest = max(lengths)
    cs, sn = plain_ops.rope_table(longest + 24, hd // 2, 1e4, 1.0, "cpu")
    scale = 1.0 / math.sqrt(hd)
    kr, vr = kc.clone(), vc.clone()
    ref = torch.empty(len(lengths), nh * hd, dtype=torch.float64)
    plain_ops.attn_decode_rope(qkv, cs, sn, kr, vr, table, pos, seq, ref, nh, nk, hd, scale, window, longest, write_kv)
    kd, vd = kc.to(DEV), vc.to(DEV)
    out = torch.empty(len(lengths), nh * hd, dtype=torch.bfloat16, device=DEV)
    ops.attn_decode_rope(qkv.to(DEV), cs.to(DEV), sn.to(DEV), kd, vd, table.to(DEV), pos.to(DEV), seq.to(DEV),
                         out, nh, nk, hd, scale, window, longest, write_kv)
    close(out, ref, 1.5e-2, 1.5e-2)
    # the cache afterwards: the own rows written (or nothing touched), everything else as before
    same = lambda a, b: torch.equal(torch.nan_to_num(a.float(), nan=7e7), torch.nan_to_num(b.float(), nan=7e7))
    if write_kv:
        close(torch.nan_to_num(kd.float(), nan=7e7), torch.nan_to_num(kr.float(), nan=7e7), 2e-2, 2e-2)
        close(torch.nan_to_num(vd.float(), nan=7e7), torch.nan_to_num(vr.float(), nan=7e7), 2e-2, 2e-2)
        for b, l in enumerate(lengths):
            page, off = int(table[b, (l - 1) // 64]), (l - 1) % 64
            assert not torch.isnan(kd[page, :, off].float()).any() and not torch.isnan(vd[page, :, off // 32, :, off % 32].float()).any()
    else:
        assert same(kd.cpu(), kc) and same(vd.cpu(), vc)


# Sequences of very unequal lengths, the longest past the length from which a step's tokens share
# its key splits in proportion to their keys (`ops.SHARED_SPLITS_FROM`).
UNEQUAL = [9000, 70, 1, 2300, 64, 129, 700, 3000]


@pytest.mark.parametrize("nh,nk,hd,window", [(8, 2, 64, 0), (28, 4, 128, 0), (6, 1, 48, 300), (4, 2, 16, 5000)])
def test_attn_tokens_splits_shared_by_length(ops, monkeypatch, nh, nk, hd, window):
    from minfer_amd.kernels import tuning
    places, splits = ops.decode_split_plan(3 * len(UNEQUAL), nk, nh // nk, max(UNEQUAL))
    assert places > splits > 1, "this case is meant to share the splits out"
    q, kc, vc, table, pos, seq = build_attention_case(nh, nk, hd, UNEQUAL, torch.bfloat16, 41)
    scale = 1.0 / math.sqrt(hd)
    ref = torch.empty(q.shape, dtype=torch.float64)
    plain_ops.attn_tokens(q, kc, vc, table, pos, seq, ref, nh, nk, hd, scale, window, max(UNEQUAL))
    dq, dk, dv, dt, dp, ds = (t.to(DEV) for t in (q, kc, vc, table, pos, seq))
    shared = torch.empty(q.shape, dtype=torch.bfloat16, device=DEV)
    ops.attn_tokens(dq, dk, dv, dt, dp, ds, shared, nh, nk, hd, scale, window, max(UNEQUAL))
    close(shared, ref, 1.5e-2, 1.5e-2)
    again = torch.full(q.shape, float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.attn_tokens(dq, dk, dv, dt, dp, ds, again, nh, nk, hd, scale, window, max(UNEQUAL))
    assert torch.equal(again, shared), "two runs differ"
    # every token with the same number of splits: the same values up to the rounding of the sums
    monkeypatch.setattr(tuning, "ATTN_EQUAL_SPLITS", True)
    assert ops.decode_split_plan(3 * len(UNEQUAL), nk, nh // nk, max(UNEQUAL)) == (splits, splits)
    equal = torch.empty(q.shape, dtype=torch.bfloat16, device=DEV)
    ops.attn_tokens(dq, dk, dv, dt, dp, ds, equal, nh, nk, hd, scale, window, max(UNEQUAL))
    close(equal, ref, 1.5e-2, 1.5e-2)
    close(shared, equal.double().cpu(), 1.5e-2, 1.5e-2)


def test_attn_tokens_shared_splits_lose_no_key(ops):
    """One key of the long sequence scaled so that its score stands out, at every place in turn where
    a split could begin or end wrongly: the output is that key's value row."""
    nh, nk, hd = 8, 8, 16
    lengths = [9000, 40, 1500, 300]
    places, splits = ops.decode_split_plan(len(lengths), nk, nh // nk, max(lengths))
    assert places > splits > 1, "this case is meant to share the splits out"
    q, kc, vc, table, _, _ = build_attention_case(nh, nk, hd, lengths, torch.bfloat16, 43)
    pos = torch.tensor([l - 1 for l in lengths], dtype=torch.int32)
    seq = torch.arange(len(lengths), dtype=torch.int32)
    q = q[:len(lengths)].clone()
    v_rows = vc.float()                      # [pages][nk][2][hd][32]
    out = torch.empty(len(lengths), nh * hd, dtype=torch.bfloat16, device=DEV)
    dv, dt, dp, ds = (t.to(DEV) for t in (vc, table, pos, seq))
    for far in (0, 127, 128, 1023, 1024, 4095, 4607, 4608, 7000, 8191, 8192, 8959, 8960, 8998, 8999):
        k = kc.clone()
        page, off = int(table[0, far // 64]), far % 64
        k[page, 0, off] = (q[0].view(nh, hd)[0].float() * 40.0).to(k.dtype)
        ops.attn_tokens(q.to(DEV), k.to(DEV), dv, dt, dp, ds, out, nh, nk, hd, 1.0, 0, max(lengths))
        want = v_rows[page, 0, off // 32, :, off % 32]
        assert torch.allclose(out[0].float().cpu().view(nh, hd)[0], want, atol=2e-2), far


@pytest.mark.parametrize("write_kv", [True, False])
@pytest.mark.parametrize("nh,nk,hd,window", [(8, 2, 64, 0), (28, 4, 128, 0), (6, 3, 48, 300)])
def test_attn_decode_rope_splits_shared_by_length(ops, nh, nk, hd, window, write_kv):
    assert ops.decode_split_plan(len(UNEQUAL), nk, nh // nk, max(UNEQUAL))[0] > \
        ops.decode_split_plan(len(UNEQUAL), nk, nh // nk, max(UNEQUAL))[1]
    decode_rope_case(ops, nh, nk, hd, window, write_kv, UNEQUAL)


def test_attention_one_key_gives_v_and_far_key_is_found(ops):
    # one key -> output = V exactly (src/graph/cpu_backend.rs:640-682), broadcast over the group
    nh, nk, hd = 4, 2, 16
    kc = torch.zeros(20, nk, 64, hd)
    vc = rnd((20, nk, 64, hd), seed=13)
    q = rnd((1, nh * hd), seed=14)
    table = torch.arange(20, dtype=torch.int32).view(1, 20)
    pos0 = torch.zeros(1, dtype=torch.int32)
    seq0 = torch.zeros(1, dtype=torch.int32)
    out = torch.empty(1, nh * hd, device=DEV)
    ops.attn_tokens(q.to(DEV), kc.to(DEV), vc.to(DEV), table.to(DEV), pos0.to(DEV), seq0.to(DEV), out,
                    nh, nk, hd, 0.25, 0, 1)
    got = out.cpu().view(nh, hd)
    for h in range(nh):
        assert torch.allclose(got[h], vc[0, h // 2, 0], atol=1e-6)
    # a far key among many: scale one key so its score stands out; output ~= its V row
    far = 777
    kc = rnd((20, nk, 64, hd), seed=15, scale=0.1)
    qv = q.view(nh, hd)
    kc[far // 64, 0, far % 64] = qv[0] * 50.0
    pos = torch.tensor([1200], dtype=torch.int32)
    ops.attn_tokens(q.to(DEV), kc.to(DEV), vc.to(DEV), table.to(DEV), pos.to(DEV), seq0.to(DEV), out,
                    nh, nk, hd, 1.0, 0, 1280)
    assert torch.allclose(out.cpu().view(nh, hd)[0], vc[far // 64, 0, far % 64], atol=1e-4)
    # the same key just outside a window is not seen, just inside it is
    for window, seen in ((1200 - far, False), (1200 - far + 1, True)):
        ops.attn_tokens(q.to(DEV), kc.to(DEV), vc.to(DEV), table.to(DEV), pos.to(DEV), seq0.to(DEV), out,
                        nh, nk, hd, 1.0, window, 1280)
        hit = torch.allclose(out.cpu().view(nh, hd)[0], vc[far // 64, 0, far % 64], atol=1e-4)
        assert hit == seen


def prefill_case(nh, nk, hd, new, start, seed):
    """Sequences that already hold start[b] tokens and bring new[b] more; caches filled for
    all of them (as the rotation kernel would have left them)."""
    from minfer_amd.engine.batch import StepContext
    rng = np.random.default_rng(seed)
    lengths = [s + n for s, n in zip(start, new)]
    n_cols = max((l + 63) // 64 for l in lengths)
    n_pages = sum((l + 63) // 64 for l in lengths) + 2
    perm = rng.permutation(n_pages)
    table = -np.ones((len(new), n_cols), dtype=np.int32)
    nxt = 0
    for b, l in enumerate(lengths):
        for c in range((l + 63) // 64):
            table[b, c] = perm[nxt]
            nxt += 1
    kc, vc = make_cache(n_pages, nk, hd, torch.bfloat16, seed)
    poison_unwritten(kc, vc, table, lengths)
    pos = torch.cat([torch.arange(s, s + n) for s, n in zip(start, new)]).int()
    seq = torch.repeat_interleave(torch.arange(len(new)), torch.tensor(new)).int()
    n_tok = int(sum(new))
    q = rnd((n_tok, nh * hd), torch.bfloat16, seed + 5)
    cu = torch.tensor([0] + list(np.cumsum(new)), dtype=torch.int32)
    table = torch.from_numpy(table)

    def ctx_on(dev):
        return StepContext(cache=None, n_tokens=n_tok, n_seqs=len(new), token_ids=torch.zeros(n_tok, dtype=torch.int32, device=dev),
                           positions=pos.to(dev), seq_of_tok=seq.to(dev), cu_seqlens=cu.to(dev),
                           start_pos=torch.tensor(start, dtype=torch.int32, device=dev),
                           slot_ids=torch.zeros(len(new), dtype=torch.int32, device=dev), logit_rows=None,
                           page_tables={}, max_len=max(lengths), max_new=max(new), all_decode=False,
                           host_new=list(new), host_start=list(start))
    return q, kc, stored_v(vc), table, ctx_on


@pytest.mark.parametrize("nh,nk,hd,window", [(4, 2, 16, 0), (4, 1, 32, 0), (9, 3, 48, 0), (28, 4, 128, 0),
                                             (6, 6, 64, 0), (10, 2, 80, 0), (4, 2, 256, 0), (4, 2, 64, 40),
                                             (7, 1, 128, 200), (4, 4, 112, 0), (12, 1, 64, 0), (130, 1, 16, 0),
                                             (2, 1, 96, 0), (2, 2, 160, 0), (3, 1, 192, 70), (2, 1, 240, 0)])
def test_attn_prefill(ops, nh, nk, hd, window):
    # new tokens per sequence straddle the blocks of queries (128 rows of (token, head of the group):
    # 128, 64, 42, 32, 25, 18 or 10 tokens; a group of 130 heads takes two workgroups a token) and the
    # 64-key pages; two sequences continue from a cache that already holds tokens
    new = [1, 5, 31, 33, 64, 65, 127, 129, 300, 70]
    start = [0, 0, 0, 0, 0, 0, 0, 0, 0, 150]
    q, kc, vc, table, ctx_on = prefill_case(nh, nk, hd, new, start, 21)
    scale = 1.0 / math.sqrt(hd)
    ref = torch.empty(q.shape, dtype=torch.float64)
    plain_ops.attn_prefill(q, kc, vc, table, ctx_on("cpu"), ref, nh, nk, hd, scale, window)
    out = torch.empty(q.shape, dtype=torch.bfloat16, device=DEV)
    ops.attn_prefill(q.to(DEV), kc.to(DEV), vc.to(DEV), table.to(DEV), ctx_on(DEV), out, nh, nk, hd, scale, window)
    close(out, ref, 1.5e-2, 1.5e-2)
    again = torch.empty(q.shape, dtype=torch.bfloat16, device=DEV)
    ops.attn_prefill(q.to(DEV), kc.to(DEV), vc.to(DEV), table.to(DEV), ctx_on(DEV), again, nh, nk, hd, scale, window)
    assert torch.equal(out, again), "two runs differ"
    # the per-token kernel gives the same answer on the same step
    tok = torch.empty(q.shape, dtype=torch.bfloat16, device=DEV)
    c = ctx_on(DEV)
    ops.attn_tokens(q.to(DEV), kc.to(DEV), vc.to(DEV), table.to(DEV), c.positions, c.seq_of_tok, tok, nh, nk, hd,
                    scale, window, c.max_len)
    close(out, tok.double(), 2e-2, 2e-2)


@pytest.mark.parametrize("nh,nk,hd,window", [(4, 2, 128, 0), (3, 1, 64, 0), (2, 2, 256, 0), (4, 1, 128, 900), (5, 5, 80, 0)])
def test_attn_prefill_shared_pages(ops, nh, nk, hd, window):
    """Long sequences with few heads: a block of queries has far more pages than a workgroup's
    share of all of them, so its pages go to up to eight workgroups in turn whose parts the last
    one adds up (one sequence continues from 600 cached tokens; the short one stays whole)."""
    new, start = [1500, 260, 40], [600, 0, 0]
    q, kc, vc, table, ctx_on = prefill_case(nh, nk, hd, new, start, 23)
    tq, gh, per_tile = ops.prefill_tile(nh, nk, hd)
    shared = ctx_on("cpu").shared_query_tiles(tq, ops.PAGE, window, per_tile, 256, 2, ops.PREFILL_MIN_PAGES,
                                              ops.PREFILL_MAX_SHARES)
    assert shared is not None
    words = shared[2].tolist()
    assert max((w >> 8) & 255 for w in words) == (8 if window == 0 else 4)     # 33 pages, or the 16 a window and a block of queries span
    by_slot = {}
    for w in words:
        if w:
            by_slot.setdefault(w >> 16, []).append((w & 255, (w >> 8) & 255))
    assert sorted(by_slot) == list(range(shared[3])) and shared[4] == max((w >> 8) & 255 for w in words)
    for got in by_slot.values():                                  # every share of a slot once
        assert sorted(s for s, _ in got) == list(range(got[0][1])) and len({n for _, n in got}) == 1
    scale = 1.0 / math.sqrt(hd)
    ref = torch.empty(q.shape, dtype=torch.float64)
    plain_ops.attn_prefill(q, kc, vc, table, ctx_on("cpu"), ref, nh, nk, hd, scale, window)
    out = torch.empty(q.shape, dtype=torch.bfloat16, device=DEV)
    ops.attn_prefill(q.to(DEV), kc.to(DEV), vc.to(DEV), table.to(DEV), ctx_on(DEV), out, nh, nk, hd, scale, window)
    close(out, ref, 1.5e-2, 1.5e-2)
    again = torch.empty(q.shape, dtype=torch.bfloat16, device=DEV)
    ops.attn_prefill(q.to(DEV), kc.to(DEV), vc.to(DEV), table.to(DEV), ctx_on(DEV), again, nh, nk, hd, scale, window)
    assert torch.equal(out, again), "two runs differ"


def test_attn_prefill_far_key_and_window_edge(ops):
    """One key's score is made to stand out for one query: the output is that key's V row
    when the key is visible (anywhere in a long prompt, across pages), and is not when the
    key lies just outside the window or after the query."""
    nh, nk, hd = 2, 1, 64
    n = 700
    q, kc, vc, table, ctx_on = prefill_case(nh, nk, hd, [n], [0], 22)
    kc = kc * 0.05
    qi, far = 650, 3
    page, row = int(table[0, far // 64]), far % 64
    kc[page, 0, row] = q[qi, :hd] * 4.0
    vrow = vc[page, 0, row // 32, :, row % 32].float()      # a bfloat16 page of V is [kv_heads][2][head_dim][32]
    for window, seen in ((0, True), (qi - far + 1, True), (qi - far, False)):
        out = torch.empty(q.shape, dtype=torch.bfloat16, device=DEV)
        ops.attn_prefill(q.to(DEV), kc.to(DEV), vc.to(DEV), table.to(DEV), ctx_on(DEV), out, nh, nk, hd, 1.0, window)
        hit = torch.allclose(out[qi, :hd].float().cpu(), vrow, atol=3e-2)
        assert hit == seen, (window, seen)
    # a query before the key never sees it
    out = torch.empty(q.shape, dtype=torch.bfloat16, device=DEV)
    q2 = q.clone()
    q2[2] = q[qi]
    ops.attn_prefill(q2.to(DEV), kc.to(DEV), vc.to(DEV), table.to(DEV), ctx_on(DEV), out, nh, nk, hd, 1.0, 0)
    assert not torch.allclose(out[2, :hd].float().cpu(), vrow, atol=3e-2)


@pytest.mark.parametrize("m,n,k", [(64, 33000, 512), (17, 32768, 256), (40, 40001, 768), (33, 152064, 256)])
def test_gemm_bf16_wide_few_rows(ops, m, n, k):
    """17..64 rows against a matrix wide enough for the whole-K kernel (a share of at least 8
    tiles for every CU; the widest takes several passes; 40001 ends inside a tile)."""
    x, w, b = rnd((m, k), torch.bfloat16, 70), rnd((n, k), torch.bfloat16, 71, 0.05), rnd((n,), seed=72)
    ref = x.double() @ w.double().t() + b.double()
    xd, wd, bd = x.to(DEV), w.to(DEV), b.to(DEV)
    tol = 2e-5 * math.sqrt(k)
    out = torch.full((m, n), 7.0, device=DEV)
    ops.linear(xd, wd, bd, out)
    close(out, ref, tol, 1e-5)
    again = torch.empty(m, n, device=DEV)
    ops.linear(xd, wd, bd, again)
    assert torch.equal(out, again)
    base = rnd((m, n), seed=73)
    acc = base.to(DEV).clone()
    ops.linear(xd, wd, None, acc, accumulate=True)
    close(acc, ref - b.double() + base.double(), tol, 1e-5)
    ob = torch.empty(m, n, dtype=torch.bfloat16, device=DEV)
    ops.linear(xd, wd, bd, ob)
    close(ob, ref, tol + 1e-3, 1e-2)


def test_tile_weight_layout(ops):
    """[n][k] -> [ceil(n / 16)][k / 32][16][32], zero rows behind n."""
    w = rnd((40, 96), torch.bfloat16, 5).to(DEV)
    t = ops.tile_weight(w)
    assert tuple(t.shape) == (3, 3, 16, 32)
    for r, k in ((0, 0), (15, 31), (16, 32), (39, 95), (17, 70)):
        assert t[r // 16, k // 32, r % 16, k % 32] == w[r, k]
    assert not t[2, :, 8:].any()
    with pytest.raises(Exception):
        ops.tile_weight(rnd((16, 40), torch.bfloat16, 6).to(DEV))


@pytest.mark.parametrize("m,n,k", [(8, 3584, 18944), (1, 1000, 8224), (16, 4608, 3584), (5, 152064, 1536),
                                   (3, 2100, 8192), (16, 8192, 8192), (8, 90, 4096), (2, 2048, 96),
                                   (8, 2100, 896), (16, 4864, 896),
                                   # 17 to 64 rows: K split over blocks, and the whole-K kernel of a wide matrix
                                   (64, 3584, 3584), (40, 3584, 18944), (17, 1000, 2048), (33, 40001, 768),
                                   (64, 33000, 512),
                                   # 17 to 64 rows and a K that is no multiple of 256: the staged kernel
                                   (40, 2048, 29568), (33, 1000, 1120), (64, 300, 96)])
def test_gemm_bf16_tiled_copy_same_bits(ops, m, n, k):
    """The products of at most 64 rows read the tiled copy of the weights where they are given one:
    the same sums in the same order, so the same bits as from the matrix itself, for every
    epilogue, with and without the folded norm; and right against the plain product."""
    x, w, b = rnd((m, k), torch.bfloat16, 120), rnd((n, k), torch.bfloat16, 121, 0.05), rnd((n,), seed=122)
    xd, wd, bd = x.to(DEV), w.to(DEV), b.to(DEV)
    wt = ops.tile_weight(wd)
    ref = x.double() @ w.double().t() + b.double()
    base = rnd((m, n), seed=123).to(DEV)
    got = []
    for tiled in (None, wt):
        out = torch.full((m, n), 7.0, device=DEV)
        ops.linear(xd, wd, bd, out, tiled=tiled)
        acc = base.clone()
        ops.linear(xd, wd, None, acc, accumulate=True, tiled=tiled)
        ob = torch.empty(m, n, dtype=torch.bfloat16, device=DEV)
        ops.linear(xd, wd, bd, ob, tiled=tiled)
        xf, g = rnd((m + 3, k), seed=124).to(DEV), rnd((k,), seed=125).to(DEV)
        idx = torch.arange(m, dtype=torch.int32, device=DEV) + 2
        on = torch.full((m, n), 7.0, device=DEV)
        folded = ops.linear_normed(xf, g, 1e-5, idx, wd, bd, on, tiled=tiled)
        got.append((out, acc, ob, on if folded else out))
    close(got[1][0], ref, 2e-5 * math.sqrt(k), 1e-5)
    for a, c in zip(*got):
        assert torch.equal(a, c)


def test_gemm_bf16_tiled_copy_moves_the_one_kernel_limit(ops):
    """9 to 12 rows against a long K: with the tiled copy the one-kernel form is the faster one,
    without it K cut over blocks and a second kernel.  Two orders of addition: both right, not
    the same bits."""
    m, n, k = 10, 3584, 18944
    assert ops.plan_linear(m, n, k)["kernel"] == "skinny_ring_kernel"
    assert ops.plan_linear(m, n, k, tiled=True)["kernel"] == "rolling16_kernel"
    x, w = rnd((m, k), torch.bfloat16, 140), rnd((n, k), torch.bfloat16, 141, 0.05)
    xd, wd = x.to(DEV), w.to(DEV)
    ref = x.double() @ w.double().t()
    for tiled in (None, ops.tile_weight(wd)):
        out = torch.empty(m, n, device=DEV)
        ops.linear(xd, wd, None, out, tiled=tiled)
        close(out, ref, 2e-5 * math.sqrt(k), 1e-5)


@pytest.mark.parametrize("m,nf,k", [(8, 18944, 3584), (1, 1024, 2048), (16, 1030, 4096), (3, 2100, 8192),
                                    (64, 18944, 512), (33, 16400, 256), (40, 300, 512)])
def test_gemm_bf16_swiglu_tiled_copy_same_bits(ops, m, nf, k):
    gate, up = rnd((nf, k), torch.bfloat16, 130, 0.05), rnd((nf, k), torch.bfloat16, 131, 0.05)
    w = ops.interleave_gate_up(gate.to(DEV), up.to(DEV))
    wt = ops.tile_weight(w)
    x = rnd((m, k), torch.bfloat16, 132).to(DEV)
    xf, g = rnd((m, k), seed=133).to(DEV), rnd((k,), seed=134).to(DEV)
    got = []
    for tiled in (None, wt):
        y = torch.empty(m, nf, dtype=torch.bfloat16, device=DEV)
        ops.linear_swiglu(x, w, y, tiled=tiled)
        yn = torch.empty(m, nf, dtype=torch.bfloat16, device=DEV)
        folded = ops.linear_normed(xf, g, 1e-6, None, w, None, yn, swiglu=True, tiled=tiled)
        got.append((y, yn if folded else y))
    for a, c in zip(*got):
        assert torch.equal(a, c)


@pytest.mark.parametrize("variant", [0, 1, 2, 9, 12, 13])
@pytest.mark.parametrize("m,nf,k", [(1, 176, 64), (8, 344, 128), (16, 32, 200), (17, 176, 64), (64, 1000, 344),
                                    (65, 232, 200), (300, 18944, 256), (130, 31, 72),
                                    (8, 1100, 1536), (3, 2100, 3584), (16, 1030, 4096), (1, 1024, 2048),
                                    (8, 1100, 5120), (3, 2100, 8192),
                                    # 17..64 rows against a wide matrix: one block per CU over the whole of K
                                    (64, 18944, 512), (33, 16400, 256), (40, 300, 512), (10, 96, 8192),
                                    # more than 64 rows but few tiles: K split over blocks
                                    (100, 1000, 1024), (200, 512, 3584)])
def test_gemm_bf16_swiglu(ops, variant, m, nf, k):
    if variant >= 12 and k % 64:
        pytest.skip("the direct-to-LDS pipeline takes k in steps of 64")
    x = rnd((m, k), torch.bfloat16, 30)
    wg, wu = rnd((nf, k), torch.bfloat16, 31, 0.3), rnd((nf, k), torch.bfloat16, 32, 0.3)
    g, u = x.double() @ wg.double().t(), x.double() @ wu.double().t()
    ref = g / (1 + torch.exp(-g)) * u
    w = ops.interleave_gate_up(wg.to(DEV), wu.to(DEV))
    assert torch.equal(w.cpu(), plain_ops.interleave_gate_up(wg, wu))
    out = torch.empty(m, nf, dtype=torch.bfloat16, device=DEV)
    ops.linear_swiglu(x.to(DEV), w, out, variant=variant)
    close(out, ref, 2e-5 * math.sqrt(k) + 1e-3, 1e-2)
    again = torch.empty(m, nf, dtype=torch.bfloat16, device=DEV)
    ops.linear_swiglu(x.to(DEV), w, again, variant=variant)
    assert torch.equal(out, again)


@pytest.mark.parametrize("m,n,k,idx", [(1, 2100, 1536, False), (5, 4608, 2048, True), (8, 4001, 3584, False),
                                       (16, 2048, 4096, True), (3, 152064, 3584, True),
                                       (2, 2100, 5120, True), (9, 5000, 5120, False), (7, 5000, 8192, True),
                                       (16, 2048, 8192, False), (1, 2100, 896, False), (8, 1152, 896, True),
                                       (16, 151936, 896, False)])
def test_gemm_bf16_normed(ops, m, n, k, idx):
    """RMS norm folded into the few-row product: against the same formula in float64 with the
    kernel's one rounding (tight), and against norm-then-product as the two kernels do it."""
    h = rnd((m + 3, k), seed=40, scale=3.0)
    h[0, 5] = 40.0                                    # one large element: the row's scale must see it
    g = 1.0 + rnd((k,), seed=41, scale=0.2)
    w, b = rnd((n, k), torch.bfloat16, 42, 0.05), rnd((n,), seed=43)
    eps = 1e-5
    row_idx = torch.tensor([(3 * i + 1) % (m + 3) for i in range(m)], dtype=torch.int32) if idx else None
    src = h if idx else h[:m].contiguous()
    ref = plain_ops.linear_normed_reference(src, g, eps, row_idx, w, b)
    out = torch.empty(m, n, device=DEV)
    done = ops.linear_normed(src.to(DEV), g.to(DEV), eps, None if row_idx is None else row_idx.to(DEV),
                             w.to(DEV), b.to(DEV), out)
    assert done, "this shape is one the folded kernel is built for"
    close(out, ref, 2e-5 * math.sqrt(k), 1e-5)
    # the two-kernel path rounds x / rms * g instead of x * g: same size of error, not the same bits
    x = torch.empty(m, k, dtype=torch.bfloat16, device=DEV)
    ops.rmsnorm(src.to(DEV), g.to(DEV), eps, x, None if row_idx is None else row_idx.to(DEV))
    two = torch.empty(m, n, device=DEV)
    ops.linear(x, w.to(DEV), b.to(DEV), two)
    exact = plain_ops.rmsnorm_reference(src if row_idx is None else src[row_idx.long()], g, eps) @ w.double().t() + b.double()
    e_fold, e_two = (out.cpu().double() - exact).abs().max().item(), (two.cpu().double() - exact).abs().max().item()
    assert e_fold <= 1.5 * e_two + 1e-4, (e_fold, e_two)
    base = rnd((m, n), seed=44)
    acc = base.to(DEV).clone()
    assert ops.linear_normed(src.to(DEV), g.to(DEV), eps, None if row_idx is None else row_idx.to(DEV),
                             w.to(DEV), None, acc, accumulate=True)
    close(acc, ref - b.double() + base.double(), 2e-5 * math.sqrt(k), 1e-5)


@pytest.mark.parametrize("m,nf,k", [(8, 1100, 1536), (3, 2100, 3584), (16, 1030, 4096), (1, 18944, 3584),
                                    (4, 2100, 5120), (16, 1100, 8192), (1, 2500, 8192), (8, 4864, 896), (16, 1100, 896)])
def test_gemm_bf16_normed_swiglu(ops, m, nf, k):
    h = rnd((m, k), seed=50, scale=2.0)
    g = 1.0 + rnd((k,), seed=51, scale=0.2)
    wg, wu = rnd((nf, k), torch.bfloat16, 52, 0.05), rnd((nf, k), torch.bfloat16, 53, 0.05)
    eps = 1e-6
    gate = plain_ops.linear_normed_reference(h, g, eps, None, wg, None)
    up = plain_ops.linear_normed_reference(h, g, eps, None, wu, None)
    ref = gate / (1 + torch.exp(-gate)) * up
    w = ops.interleave_gate_up(wg.to(DEV), wu.to(DEV))
    out = torch.empty(m, nf, dtype=torch.bfloat16, device=DEV)
    assert ops.linear_normed(h.to(DEV), g.to(DEV), eps, None, w, None, out, swiglu=True)
    close(out, ref, 2e-5 * math.sqrt(k) + 1e-3, 1e-2)


def test_gemm_bf16_normed_declines(ops):
    """Shapes without a folded kernel: nothing is written and the caller is told."""
    h, g = rnd((4, 200), seed=60), rnd((200,), seed=61)
    w = rnd((300, 200), torch.bfloat16, 62)
    out = torch.full((4, 300), 7.0, device=DEV)
    assert not ops.linear_normed(h.to(DEV), g.to(DEV), 1e-6, None, w.to(DEV), None, out)
    assert not ops.linear_normed(rnd((17, 2048), seed=63).to(DEV), rnd((2048,), seed=64).to(DEV), 1e-6, None,
                                 rnd((4096, 2048), torch.bfloat16, 65).to(DEV), None,
                                 torch.full((17, 4096), 7.0, device=DEV))
    torch.cuda.synchronize()
    assert torch.all(out == 7.0)


# ------------------------------------------------------------------ the norm folded around the products of at most 64 rows
@pytest.mark.parametrize("m,n,k", [(64, 3584, 3584), (20, 3584, 18944), (33, 5120, 5120), (17, 1000, 2048), (64, 3584 + 24, 3584),
                                   (8, 3584, 3584), (16, 3584, 18944), (1, 3584, 18944), (5, 896, 4864), (13, 2048, 11008),
                                   (8, 5120, 5120), (3, 1536, 1536)])
def test_product_prepares_the_next_norm(ops, m, n, k):
    """A product that adds into the residual stream and leaves, for the norm that reads the stream
    next, bf16(stream g) and the rows' sums of squares in parts (runs of 256 columns from 17 rows on,
    one part per workgroup of the one-kernel forms below that, the unused places zero): the stream
    itself is what `linear` gives bit for bit, and what it leaves is what the stream's new rows say."""
    x, w, b = rnd((m, k), torch.bfloat16, 70), rnd((n, k), torch.bfloat16, 71, 0.05), rnd((n,), seed=72)
    g = (1.0 + rnd((n,), seed=73, scale=0.2)).to(DEV)
    base = rnd((m, n), seed=74, scale=3.0)
    base[m - 1, 7] = 50.0
    plain = base.to(DEV).clone()
    ops.linear(x.to(DEV), w.to(DEV), b.to(DEV), plain, accumulate=True)
    out = base.to(DEV).clone()
    xg = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEV)
    sums = torch.full((m, ops.norm_sum_parts(n, m)), float("nan"), device=DEV)
    tiled = ops.tile_weight(w.to(DEV)) if m <= 16 else None
    assert ops.linear_fused(x.to(DEV), w.to(DEV), b.to(DEV), out, accumulate=True, norm_out=(g, xg, sums), tiled=tiled)
    assert torch.equal(out, plain)
    assert torch.equal(xg, (out * g).to(torch.bfloat16))
    if m > 16:
        want = torch.nn.functional.pad(out.double() ** 2, (0, sums.shape[1] * 256 - n)).view(m, -1, 256).sum(-1)
        close(sums, want.cpu(), 1e-6 * float(want.max()), 1e-5)
    else:
        assert torch.isfinite(sums).all() and (sums >= 0).all()
        want = (out.double() ** 2).sum(-1)
        close(sums.double().sum(-1), want.cpu(), 1e-6 * float(want.max()), 1e-5)
    # twice the same bits
    xg2, sums2, out2 = torch.empty_like(xg), torch.empty_like(sums), base.to(DEV).clone()
    assert ops.linear_fused(x.to(DEV), w.to(DEV), b.to(DEV), out2, accumulate=True, norm_out=(g, xg2, sums2), tiled=tiled)
    assert torch.equal(xg, xg2) and torch.equal(sums, sums2) and torch.equal(out, out2)


@pytest.mark.parametrize("m,n,k,swiglu", [(64, 4608, 3584, False), (20, 37888, 3584, True), (40, 152064, 3584, False),
                                          (33, 7168, 5120, False), (17, 1000, 2048, False), (64, 2200, 2048, True),
                                          (8, 4608, 3584, False), (16, 37888, 3584, True), (1, 152064, 3584, False),
                                          (5, 1152, 896, False), (7, 9728, 896, True), (12, 7168, 5120, False),
                                          (3, 22016, 2048, True)])
def test_product_takes_a_prepared_norm(ops, m, n, k, swiglu):
    """The product behind the norm: its activations are bf16(x g), its sums are multiplied by each
    row's 1 / sqrt(sum of the partial sums / k + eps).  Against the formula in float64 with that one
    rounding, and against norm-then-product as the two kernels do it (the same size of error)."""
    h = rnd((m, k), seed=80, scale=3.0)
    h[min(2, m - 1), 11] = 45.0
    gw = 1.0 + rnd((k,), seed=81, scale=0.2)
    eps = 1e-5
    xg = (h * gw).to(torch.bfloat16).to(DEV)
    parts = ops.norm_sum_parts(k)
    sums = torch.nn.functional.pad(h.double() ** 2, (0, parts * 256 - k)).view(m, parts, 256).sum(-1).float().to(DEV)
    if m <= 16:         # as a one-kernel product leaves them: a part per workgroup, zeros behind the last
        sums = torch.nn.functional.pad(sums, (0, ops.norm_sum_parts(k, m) - parts))
    if swiglu:
        nf = n // 2
        wg, wu = rnd((nf, k), torch.bfloat16, 82, 0.05), rnd((nf, k), torch.bfloat16, 83, 0.05)
        gate = plain_ops.linear_normed_reference(h, gw, eps, None, wg, None)
        up = plain_ops.linear_normed_reference(h, gw, eps, None, wu, None)
        ref = gate / (1 + torch.exp(-gate)) * up
        out = torch.empty(m, nf, dtype=torch.bfloat16, device=DEV)
        assert ops.linear_fused(xg, ops.interleave_gate_up(wg.to(DEV), wu.to(DEV)), None, out, swiglu=True, scale_in=(sums, eps))
        close(out, ref, 2e-5 * math.sqrt(k) + 1e-3, 1e-2)
        return
    w, b = rnd((n, k), torch.bfloat16, 84, 0.05), rnd((n,), seed=85)
    ref = plain_ops.linear_normed_reference(h, gw, eps, None, w, b)
    out = torch.empty(m, n, device=DEV)
    assert ops.linear_fused(xg, w.to(DEV), b.to(DEV), out, scale_in=(sums, eps))
    close(out, ref, 2e-5 * math.sqrt(k), 1e-5)
    x = torch.empty(m, k, dtype=torch.bfloat16, device=DEV)
    ops.rmsnorm(h.to(DEV), gw.to(DEV), eps, x)
    two = torch.empty(m, n, device=DEV)
    ops.linear(x, w.to(DEV), b.to(DEV), two)
    exact = plain_ops.rmsnorm_reference(h, gw, eps) @ w.double().t() + b.double()
    e_fold, e_two = (out.cpu().double() - exact).abs().max().item(), (two.cpu().double() - exact).abs().max().item()
    assert e_fold <= 1.5 * e_two + 1e-4, (e_fold, e_two)
    base = rnd((m, n), seed=86)
    acc = base.to(DEV).clone()
    assert ops.linear_fused(xg, w.to(DEV), None, acc, accumulate=True, scale_in=(sums, eps))
    close(acc, ref - b.double() + base.double(), 2e-5 * math.sqrt(k), 1e-5)


def test_fused_norm_declines_where_no_kernel_has_a_place_for_it(ops):
    """A K that is not split at 17 rows and more, a shape of few rows that the register-resident
    kernel does not take: nothing is written, the caller is told."""
    for m, n, k in ((8, 300, 200), (20, 300, 200), (64, 64, 256)):
        x, w = rnd((m, k), torch.bfloat16, 90).to(DEV), rnd((n, k), torch.bfloat16, 91).to(DEV)
        out = torch.full((m, n), 7.0, device=DEV)
        xg = torch.full((m, n), 3.0, dtype=torch.bfloat16, device=DEV)
        sums = torch.full((m, ops.norm_sum_parts(n, m)), 5.0, device=DEV)
        g = torch.ones(n, device=DEV)
        assert not ops.linear_fused(x, w, None, out, accumulate=True, norm_out=(g, xg, sums))
        s_in = torch.ones((m, ops.norm_sum_parts(k)), device=DEV)
        assert not ops.linear_fused(x, w, None, out, scale_in=(s_in, 1e-6))
        torch.cuda.synchronize()
        assert torch.all(out == 7.0) and torch.all(xg == 3.0) and torch.all(sums == 5.0)

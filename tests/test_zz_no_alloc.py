"""The entry point that allocates nothing (csrc/noalloc.h), called through ctypes: the same
output as the entry point that takes the caller's workspace, on two calls in a row of which the
second is smaller (so it finds the first one's partials in the library's array), both against
plain attention in 64 bits, a size beyond the array refused, and the device's free memory (the
driver's figure, not torch's) the same before and after a call."""
import ctypes
from ctypes import c_float, c_int, c_size_t, c_void_p

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
PAGE = 64
TOO_LARGE = -3


def library():
    from minfer_amd.kernels import build
    lib = build.load("attn_decode_bf16")
    P = c_void_p
    lib.mf_attn_decode_bf16.argtypes = [P, P, P, P, c_int, P, P, P, P, c_int, c_int, c_int, c_int, c_float, c_int,
                                        c_int, c_int, P]
    lib.mf_attn_decode_bf16.restype = c_int
    lib.mf_attn_decode_bf16_noalloc.argtypes = [P, P, P, P, c_int, P, P, P, c_int, c_int, c_int, c_int, c_float,
                                                c_int, c_int, P]
    lib.mf_attn_decode_bf16_noalloc.restype = c_int
    lib.mf_attn_decode_bf16_noalloc_capacity.argtypes = []
    lib.mf_attn_decode_bf16_noalloc_capacity.restype = c_size_t
    return lib


def case(n_seq, lengths, nh, nk, hd, seed):
    """Random queries, and a paged cache whose pages are dealt out in a shuffled order."""
    g = torch.Generator().manual_seed(seed)
    n_pages_seq = [(n + PAGE - 1) // PAGE for n in lengths]
    total = sum(n_pages_seq) + 3
    order = torch.randperm(total, generator=g).tolist()
    cols = max(n_pages_seq)
    table = torch.full((n_seq, cols), -1, dtype=torch.int32)
    for b, n in enumerate(n_pages_seq):
        for c in range(n):
            table[b, c] = order.pop()
    kc = (torch.randn(total, nk, PAGE, hd, generator=g) * 0.5).to(torch.bfloat16)
    vt = (torch.randn(total, nk, 2, hd, PAGE // 2, generator=g) * 0.5).to(torch.bfloat16)
    q = (torch.randn(n_seq, nh * hd, generator=g) * 0.5).to(torch.bfloat16)
    pos = torch.tensor([n - 1 for n in lengths], dtype=torch.int32)
    seq = torch.arange(n_seq, dtype=torch.int32)
    return [t.to(DEV) for t in (q, kc, vt, table, pos, seq)]


def run_both(lib, tensors, nh, nk, hd, n_splits, scale=0.11):
    q, kc, vt, table, pos, seq = tensors
    n_tok = q.shape[0]
    stream = c_void_p(torch.cuda.current_stream().cuda_stream)
    p = lambda t: c_void_p(t.data_ptr())
    want = torch.full((n_tok, nh * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
    got = torch.full_like(want, float("nan"))
    part = torch.empty(max(1, n_tok * nh * n_splits * (hd + 2)), dtype=torch.float32, device=DEV)
    rc = lib.mf_attn_decode_bf16(p(q), p(kc), p(vt), p(table), table.shape[1], p(pos), p(seq), p(want), p(part),
                                 n_tok, nh, nk, hd, scale, 0, n_splits, 0, stream)
    assert rc == 0
    torch.cuda.synchronize()
    # what the device itself has free (the driver's figure, which a hipMalloc inside the library
    # would move; torch's own counters see only torch's allocator) and what torch has reserved
    free_before, reserved_before = torch.cuda.mem_get_info(DEV)[0], torch.cuda.memory_reserved(DEV)
    rc = lib.mf_attn_decode_bf16_noalloc(p(q), p(kc), p(vt), p(table), table.shape[1], p(pos), p(seq), p(got),
                                         n_tok, nh, nk, hd, scale, 0, n_splits, stream)
    assert rc == 0, f"noalloc entry point returned {rc}"
    torch.cuda.synchronize()
    assert torch.cuda.memory_reserved(DEV) == reserved_before
    assert torch.cuda.mem_get_info(DEV)[0] == free_before, "the call changed the device's free memory"
    return want, got


def plain_attention(tensors, nh, nk, hd, scale=0.11):
    """softmax(q.k scale) v in 64 bits from the pages, one head at a time: [tokens][heads * hd]."""
    q, kc, vt, table, pos, seq = [t.cpu() for t in tensors]
    out = torch.zeros(q.shape, dtype=torch.float64)
    for b in range(q.shape[0]):
        n = int(pos[b]) + 1
        pages = table[int(seq[b]), :(n + PAGE - 1) // PAGE].long()
        k = kc[pages].double().permute(1, 0, 2, 3).reshape(nk, -1, hd)[:, :n]                 # [nk][keys][hd]
        v = vt[pages].double().permute(1, 0, 2, 4, 3).reshape(nk, -1, hd)[:, :n]              # [pages][nk][2][hd][32] -> keys
        qh = q[b].double().view(nh, hd)
        for h in range(nh):
            s = (k[h // (nh // nk)] @ qh[h]) * scale
            out[b, h * hd:(h + 1) * hd] = torch.softmax(s, 0) @ v[h // (nh // nk)]
    return out


def close_to_plain(got, tensors, nh, nk, hd):
    """Against plain attention in 64 bits, so that "equal" is not "equally wrong": the output is
    rounded to bfloat16 (values up to about 1) and the probabilities are before the second product."""
    want = plain_attention(tensors, nh, nk, hd)
    err = (got.double().cpu() - want).abs().max().item()
    assert err < 2e-2, err


def test_noalloc_entry_point_matches_the_workspace_one_twice_in_a_row():
    lib = library()
    assert lib.mf_attn_decode_bf16_noalloc_capacity() == 1 << 20
    nh, nk, hd = 28, 4, 128
    # a first, small call, so that the library's set-up (the address of its array) is behind us
    # when free memory is compared around the calls below
    run_both(lib, case(1, [70], nh, nk, hd, seed=9), nh, nk, hd, n_splits=2)
    # first call: 6 sequences of up to 2,000 keys in 8 splits; second: fewer, shorter, fewer splits,
    # so the array still holds the first call's partials beyond and between what the second writes
    first = case(6, [2000, 1300, 777, 64, 65, 1], nh, nk, hd, seed=1)
    want, got = run_both(lib, first, nh, nk, hd, n_splits=8)
    assert torch.isfinite(want.float()).all() and torch.equal(want, got)
    close_to_plain(got, first, nh, nk, hd)
    second = case(2, [300, 129], nh, nk, hd, seed=2)
    want2, got2 = run_both(lib, second, nh, nk, hd, n_splits=3)
    assert torch.isfinite(want2.float()).all() and torch.equal(want2, got2)
    close_to_plain(got2, second, nh, nk, hd)
    # one split: no scratch at all
    want3, got3 = run_both(lib, second, nh, nk, hd, n_splits=1)
    assert torch.equal(want3, got3)
    close_to_plain(got3, second, nh, nk, hd)
    # other head sizes and groups go through the same kernels
    third = case(3, [500, 31, 260], 9, 3, 48, seed=3)
    want4, got4 = run_both(lib, third, 9, 3, 48, n_splits=4)
    assert torch.equal(want4, got4)
    close_to_plain(got4, third, 9, 3, 48)


def test_noalloc_entry_point_refuses_what_its_array_cannot_hold():
    lib = library()
    nh, nk, hd = 28, 4, 128
    tensors = case(2, [100, 90], nh, nk, hd, seed=4)
    q, kc, vt, table, pos, seq = tensors
    out = torch.zeros_like(q)
    p = lambda t: c_void_p(t.data_ptr())
    stream = c_void_p(torch.cuda.current_stream().cuda_stream)
    # 2 tokens fit; pretend there are 600 (the host check comes before anything is read)
    need = 600 * nh * 32 * (hd + 2)
    assert need > (1 << 20)
    rc = lib.mf_attn_decode_bf16_noalloc(p(q), p(kc), p(vt), p(table), table.shape[1], p(pos), p(seq), p(out),
                                         600, nh, nk, hd, 0.1, 0, 32, stream)
    assert rc == TOO_LARGE
    torch.cuda.synchronize()
    assert not out.any(), "a refused call launches nothing"
    rc = lib.mf_attn_decode_bf16_noalloc(p(q), p(kc), p(vt), p(table), table.shape[1], p(pos), p(seq), p(out),
                                         2, nh, nk, hd, 0.1, 0, 65, stream)
    assert rc == 1                                                     # hipErrorInvalidValue: at most 64 splits

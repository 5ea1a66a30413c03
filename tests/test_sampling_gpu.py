"""The sampling kernels against the plain sampler (tests/plain_qwen2.py)."""
import numpy as np
import pytest
import torch

import plain_qwen2 as pq
from minfer_amd.sampling import Sampler, SamplingParams, stream_i64, uniform

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def streams_of(seed, keys):
    """Stream ids (seed and key folded on the host) as the int64 tensor the kernels read."""
    return torch.tensor([stream_i64(seed, k) for k in keys], dtype=torch.int64, device=DEV)


@pytest.fixture(scope="module")
def ops():
    from minfer_amd.kernels import ops as o
    return o


def logits_rows(rows, vocab, seed, scale=3.0):
    return (torch.randn(rows, vocab, generator=torch.Generator().manual_seed(seed)) * scale).float()


@pytest.mark.parametrize("rows,vocab", [(1, 4), (5, 1000), (3, 152064), (64, 777)])
def test_argmax_first_maximum(ops, rows, vocab):
    l = logits_rows(rows, vocab, 1)
    l[0, vocab // 2] = l[0, vocab - 1] = 50.0                 # a tie: the lower index wins
    out = torch.empty(rows, dtype=torch.int32, device=DEV)
    ops.argmax(l.to(DEV), out)
    assert out.cpu().tolist() == [pq.greedy(r.numpy()) for r in l]
    assert out[0].item() == vocab // 2


def test_reference_vectors(ops):
    def run(fn, vals, *a):
        t = torch.tensor([vals], dtype=torch.float32, device=DEV)
        fn(t, *a)
        return t.cpu()[0].tolist()
    out = torch.empty(1, dtype=torch.int32, device=DEV)
    ops.argmax(torch.tensor([[1., 5, -2, 3]], device=DEV), out)
    assert out.item() == 1                                                    # src/sampler.rs:313-317
    k = run(ops.top_k, [1., 5, 2, 4], 2)
    assert k[1] == 5 and k[3] == 4 and k[0] == k[2] == float("-inf")           # :344-351
    p = run(ops.top_p, [1., 2, 3, 4], 0.5)
    assert p[3] == 4.0 and all(v == float("-inf") for v in p[:3])              # :354-363
    prev = torch.tensor([[3, 3, 0, 0]], dtype=torch.int32, device=DEV)
    n1, n2 = (torch.tensor([n], dtype=torch.int32, device=DEV) for n in (1, 2))
    assert run(ops.penalties, [1., 2, 3, 4], prev, n1, 2.0, 0.0, 0.0)[3] == 2.0      # :320-333
    assert run(ops.penalties, [-4., -2, -1, -3], prev, n1, 2.0, 0.0, 0.0)[3] == -6.0
    assert run(ops.penalties, [1., 2, 3, 4], prev, n2, 1.0, 0.5, 0.0) == [1, 2, 3, 3]  # :388-397
    assert abs(run(ops.penalties, [1., 2, 3, 4], prev, n2, 1.0, 0.0, 0.8)[3] - 3.2) < 1e-6
    prev0 = torch.tensor([[0, 99]], dtype=torch.int32, device=DEV)
    assert run(ops.penalties, [4., -4, 0, 0], prev0, n2, 2.0, 1.0, 1.0) == [1, -4, 0, 0]  # :411-427, :448-452


@pytest.mark.parametrize("vocab,k", [(1000, 40), (152064, 40), (777, 1), (50, 49), (3000, 700)])
def test_top_k_matches_plain(ops, vocab, k):
    l = logits_rows(4, vocab, 2)
    l[1, :50] = 1.25                                           # many ties around the threshold
    d = l.to(DEV).clone()
    ops.top_k(d, k)
    for i in range(4):
        assert np.array_equal(d[i].cpu().numpy(), pq.apply_top_k(l[i].numpy(), k))


@pytest.mark.parametrize("vocab,p,pre_k", [(1000, 0.95, 40), (152064, 0.95, 40), (500, 0.5, 0), (4000, 0.9, 0),
                                           (64, 0.3, 0)])
def test_top_p_matches_plain(ops, vocab, p, pre_k):
    l = logits_rows(4, vocab, 3)
    l[2, :10] = 2.0                                            # equal probabilities: index order decides
    if pre_k:
        l = torch.stack([torch.from_numpy(pq.apply_top_k(r.numpy(), pre_k)) for r in l])
    d = l.to(DEV).clone()
    ops.top_p(d, p)
    for i in range(4):
        want = pq.apply_top_p(l[i].numpy(), p)
        got = d[i].cpu().numpy()
        if not np.array_equal(got, want):
            # the two may differ by one element only when the cumulative mass touches p within rounding
            kept_w, kept_g = np.isfinite(want), np.isfinite(got)
            assert abs(int(kept_w.sum()) - int(kept_g.sum())) <= 1
            probs = torch.softmax(l[i].double(), 0).numpy()
            assert abs(min(probs[kept_w].sum(), probs[kept_g].sum()) - p) < 1e-5


@pytest.mark.parametrize("vocab,temp", [(100, 0.8), (152064, 0.8), (777, 1.3), (1000, 0.05)])
def test_temperature_draw_matches_plain(ops, vocab, temp):
    rows = 16
    l = logits_rows(rows, vocab, 4)
    if vocab == 100:
        l = (torch.arange(100).float() * 0.1).repeat(rows, 1)              # src/sampler.rs:366-375
    rs = np.random.default_rng(5).random(rows).astype(np.float32)
    rs[0], rs[1] = 0.0, 0.99999994
    out = torch.empty(rows, dtype=torch.int32, device=DEV)
    keys = torch.zeros(rows, dtype=torch.int64, device=DEV)
    steps = torch.zeros(rows, dtype=torch.int32, device=DEV)
    ops.sample(l.to(DEV), temp, keys, steps, out, torch.from_numpy(rs).to(DEV))
    for i in range(rows):
        probs = pq.temperature_probs(l[i].numpy(), temp)
        # the kernel keeps the running sum in double; so does the oracle for a large vocabulary
        # (the reference's f32 running sum drifts by ~1e-4 over 10^5 entries)
        acc = np.float32 if vocab <= 1000 else np.float64
        want, got = pq.sample_from_probs(probs, float(rs[i]), acc), int(out[i])
        if want != got:          # only when the draw is within rounding of the running sum at both
            cum = np.cumsum(probs.astype(np.float64))
            assert abs(cum[got] - rs[i]) < 1e-6 and abs(cum[want] - rs[i]) < 1e-6, (i, want, got)
    # masked entries are never drawn
    m = torch.full((1, 50), float("-inf"))
    m[0, 7] = m[0, 31] = 1.0
    for r, want in ((0.0, 7), (0.49, 7), (0.51, 31), (0.999, 31)):
        ops.sample(m.to(DEV), 1.0, keys[:1], steps[:1], out[:1], torch.tensor([r], device=DEV))
        assert out[0].item() == want


@pytest.mark.parametrize("rows,vocab,k,p,temp", [(8, 152064, 40, 0.95, 0.8), (6, 1000, 40, 0.9, 0.7),
                                                 (5, 777, 1, 0.55, 1.3), (6, 5000, 48, 1.0, 0.8),
                                                 (5, 300, 40, 0.95, 0.8), (64, 32000, 20, 0.8, 1.0)])
def test_sample_filtered_is_top_k_top_p_and_the_draw(ops, rows, vocab, k, p, temp):
    """The fused kernels give the tokens of the three whole-row kernels one after the other, with
    ties at the k-th value, with fewer finite entries than k, and for a constant row (more equal
    values than the lists hold: the whole-row kernels run inside); they leave the logits alone
    where they can."""
    l = logits_rows(rows, vocab, 11)
    l[1, :50] = 9.0                                            # ties that reach into the k largest
    l[2] = float("-inf")
    l[2, [3, vocab // 2, vocab - 1]] = torch.tensor([0.5, 1.5, 1.0])     # fewer finite entries than k
    l[3] = 0.25                                                # a constant row
    rs = np.random.default_rng(12).random(rows).astype(np.float32)
    rs[0], rs[4] = 0.0, 0.99999994
    forced = torch.from_numpy(rs).to(DEV)
    keys = torch.zeros(rows, dtype=torch.int64, device=DEV)
    steps = torch.zeros(rows, dtype=torch.int32, device=DEV)
    chain = l.to(DEV).clone()
    want = torch.empty(rows, dtype=torch.int32, device=DEV)
    ops.top_k(chain, k)
    ops.top_p(chain, p)
    ops.sample(chain, temp, keys, steps, want, forced)
    d = l.to(DEV).clone()
    got = torch.empty(rows, dtype=torch.int32, device=DEV)
    assert ops.sample_filtered_takes(vocab, k, temp)
    ops.sample_filtered(d, k, p, temp, keys, steps, got, forced)
    assert got.cpu().tolist() == want.cpu().tolist()
    untouched = [i for i in range(rows) if i != 3]
    assert torch.equal(d[untouched].cpu(), l[untouched])
    # and the tokens are the plain sampler's (but for the constant row, where a walk over the
    # whole vocabulary in 32 bits, as the plain sampler does it, drifts, and for the draw next to 1,
    # where the last bit of the probabilities' sum decides between the last kept token and the
    # fallback)
    for i in untouched:
        if i != 4:
            assert int(got[i]) == pq.sample(l[i].numpy(), temp, float(rs[i]), k, p, 1.0, 0.0, 0.0, [])
    # without forced draws: the generator's uniform, as `sample` takes it
    keys = streams_of(77, range(5, rows + 5))
    steps = torch.arange(rows, dtype=torch.int32, device=DEV)
    chain = l.to(DEV).clone()
    ops.top_k(chain, k)
    ops.top_p(chain, p)
    ops.sample(chain, temp, keys, steps, want)
    ops.sample_filtered(l.to(DEV).clone(), k, p, temp, keys, steps, got)
    assert got.cpu().tolist() == want.cpu().tolist()


def test_sample_filtered_with_many_candidates(ops):
    """A row whose pieces' maxima bound its k-th largest entry loosely: the 40 largest sit in one
    piece, every other piece has a dozen entries at its own maximum, which is the bound, so the
    lists hold some 800 candidates for 40 survivors (more than find their places by counting: the
    lists' heads are taken one by one).  A second row with 300 candidates takes the counting."""
    vocab, k, p, temp = 152064, 40, 0.95, 0.8
    per = (vocab + 63) // 64
    l = logits_rows(2, vocab, 21).clamp(-1.0, 1.0)
    for row, dozen in ((0, 12), (1, 4)):
        l[row, 100:100 + k] = 10.0 + 0.01 * torch.arange(k)
        for piece in range(1, 64):
            l[row, piece * per + 7 * torch.arange(dozen)] = 5.0
    rs = torch.tensor([0.3, 0.97], device=DEV)
    keys = torch.zeros(2, dtype=torch.int64, device=DEV)
    steps = torch.zeros(2, dtype=torch.int32, device=DEV)
    chain = l.to(DEV).clone()
    want = torch.empty(2, dtype=torch.int32, device=DEV)
    ops.top_k(chain, k)
    ops.top_p(chain, p)
    ops.sample(chain, temp, keys, steps, want, rs)
    d = l.to(DEV).clone()
    got = torch.empty(2, dtype=torch.int32, device=DEV)
    ops.sample_filtered(d, k, p, temp, keys, steps, got, rs)
    assert got.cpu().tolist() == want.cpu().tolist()
    assert all(100 <= t < 100 + k for t in got.cpu().tolist())
    assert torch.equal(d.cpu(), l)


def test_device_uniform_is_the_host_uniform_and_draws_follow_softmax(ops):
    rows, vocab = 4000, 3
    small = torch.tensor([0.0, 1.0, 2.0]).repeat(rows, 1).to(DEV)
    keys = streams_of(42, range(rows))
    steps = (torch.arange(rows, dtype=torch.int32, device=DEV) % 7)
    out = torch.empty(rows, dtype=torch.int32, device=DEV)
    ops.sample(small, 1.0, keys, steps, out)
    probs = pq.temperature_probs(np.array([0, 1, 2], dtype=np.float32), 1.0)
    want = [pq.sample_from_probs(probs, uniform(42, i, i % 7)) for i in range(rows)]
    assert out.cpu().tolist() == want
    counts = np.bincount(out.cpu().numpy(), minlength=3)
    expect = probs * rows
    assert (np.abs(counts - expect) < 4 * np.sqrt(expect)).all()


def test_pipeline_order_and_greedy_with_penalty():
    l = torch.tensor([[1., 2, 3, 4]], device=DEV)
    out = torch.empty(1, dtype=torch.int32, device=DEV)
    keys, steps = torch.zeros(1, dtype=torch.int64, device=DEV), torch.zeros(1, dtype=torch.int32, device=DEV)
    prev, n = torch.tensor([[3]], dtype=torch.int32, device=DEV), torch.ones(1, dtype=torch.int32, device=DEV)
    Sampler(SamplingParams(temp=0.0, repeat_penalty=2.0))(l, keys, steps, out, prev, n)
    assert out.item() == 2                                                  # src/sampler.rs:378-383
    rows, vocab = 8, 5000
    base = logits_rows(rows, vocab, 6)
    params = SamplingParams(temp=0.7, top_k=40, top_p=0.9, repeat_penalty=1.3, frequency_penalty=0.2,
                            presence_penalty=0.1, seed=9)
    windows = [[int(t) for t in np.random.default_rng(i).integers(0, vocab, size=20)] for i in range(rows)]
    prev = torch.zeros(rows, 64, dtype=torch.int32)
    for i, w in enumerate(windows):
        w[0] = int(torch.argmax(base[i]))                  # penalise the favourite
        prev[i, :20] = torch.tensor(w)
    out = torch.empty(rows, dtype=torch.int32, device=DEV)
    sampler = Sampler(params)
    sampler(base.to(DEV).clone(), torch.tensor(sampler.streams(range(rows)), dtype=torch.int64, device=DEV),
                    torch.full((rows,), 3, dtype=torch.int32, device=DEV), out, prev.to(DEV),
                    torch.full((rows,), 20, dtype=torch.int32, device=DEV))
    want = [pq.sample(base[i].numpy(), 0.7, uniform(9, i, 3), 40, 0.9, 1.3, 0.2, 0.1, windows[i]) for i in range(rows)]
    assert out.cpu().tolist() == want


def test_advance_feeds_back_and_keeps_the_recent_window(ops):
    """After a step the sampled token is the next input, positions and steps move on, and the
    token enters the window of recent tokens: appended while there is room, over the oldest
    afterwards; the penalties then see exactly the last `window` tokens."""
    import plain_ops
    n, window = 3, 4
    next_ids = torch.zeros(n, dtype=torch.int32)
    positions = torch.tensor([5, 0, 70], dtype=torch.int32)
    steps = torch.tensor([1, 0, 9], dtype=torch.int32)
    prev = torch.zeros(n, window, dtype=torch.int32)
    prev[0, :2] = torch.tensor([7, 8], dtype=torch.int32)
    prev[2] = torch.tensor([1, 2, 3, 4], dtype=torch.int32)
    n_prev = torch.tensor([2, 0, 4], dtype=torch.int32)
    cursor = torch.tensor([2, 0, 0], dtype=torch.int32)
    dev = [t.to(DEV) for t in (next_ids, positions, steps, prev, n_prev, cursor)]
    cpu = [t.clone() for t in (next_ids, positions, steps, prev, n_prev, cursor)]
    history = [[7, 8], [], [1, 2, 3, 4]]
    for step in range(6):
        sampled = torch.tensor([10 + step, 20 + step, 30 + step], dtype=torch.int32)
        ops.advance(dev[0], sampled.to(DEV), dev[1], dev[2], dev[3], dev[4], dev[5])
        plain_ops.advance(cpu[0], sampled, cpu[1], cpu[2], cpu[3], cpu[4], cpu[5])
        for a, b in zip(dev, cpu):
            assert torch.equal(a.cpu(), b)
        for i in range(n):
            history[i].append(int(sampled[i]))
            got = sorted(dev[3][i, :int(dev[4][i])].cpu().tolist())
            assert got == sorted(history[i][-window:])
    assert dev[0].cpu().tolist() == [15, 25, 35] and dev[1].cpu().tolist() == [11, 6, 76]
    # without a window nothing but ids, positions and steps is touched
    ops.advance(dev[0], dev[0].clone(), dev[1], dev[2])
    assert dev[1].cpu().tolist() == [12, 7, 77]

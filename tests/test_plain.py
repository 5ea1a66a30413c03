"""Pins of the plain implementation beside the reference's text: vectors that the
reference's own tests hold, special cases that reduce to a library routine, invariants.
Each is chosen so that a plausible mistake (a wrong sign or pairing, eps or a norm in the
wrong place, a wrong head mapping) fails it."""
import math

import numpy as np
import pytest
import torch

import plain_qwen2 as pq
from minfer_amd import config_from_dict
from tiny import TINIES, random_tokens, write_tiny


def rnd(*shape, seed=0):
    return np.random.default_rng(seed).standard_normal(shape)


# ------------------------------------------------------------------ linear, silu
def test_linear_bias_silu_reference_vector():
    # src/graph/cpu_backend.rs:540-566
    w = np.array([[1., 0, 0, 0], [0, 2, 0, 0], [0, 0, 3, 0]])
    y = pq.linear(np.array([[1., 2, 3, 4]]), w, np.array([0.5, -1.0, 0.25]))
    assert y.tolist() == [[1.5, 3.0, 9.25]]
    s = lambda v: v / (1 + math.exp(-v))
    assert np.allclose(pq.silu(y) * 2, [[2 * s(1.5), 2 * s(3.0), 2 * s(9.25)]], atol=1e-12)
    x, wr, b = rnd(5, 7, seed=1), rnd(3, 7, seed=2), rnd(3, seed=3)
    assert np.allclose(pq.linear(x, wr, b), torch.nn.functional.linear(torch.tensor(x), torch.tensor(wr), torch.tensor(b)).numpy())


def test_silu_limits_and_library():
    z = np.array([0.0, 50.0, -50.0, 88.0, -88.0, 1.3])
    y = pq.silu(z)
    assert y[0] == 0 and abs(y[1] - 50) < 1e-12 and abs(y[2]) < 1e-12 and np.isfinite(y).all()
    assert np.allclose(y, torch.nn.functional.silu(torch.tensor(z)).numpy())
    x = rnd(4, 6, seed=4)
    wg, wu, wd = rnd(9, 6, seed=5), rnd(9, 6, seed=6), rnd(6, 9, seed=7)
    t = lambda a: torch.tensor(a)
    lib = torch.nn.functional.linear(torch.nn.functional.silu(t(x) @ t(wg).T) * (t(x) @ t(wu).T), t(wd))
    assert np.allclose(pq.swiglu_ffn(x, wg, wu, wd), lib.numpy())


# ------------------------------------------------------------------ RMSNorm
def test_rmsnorm_reference_vectors():
    # src/graph/cpu_backend.rs:569-594: rows [1,2,3,4] and [.5,-.5,2,-3], w = 1, eps 1e-5
    x = np.array([[1., 2, 3, 4], [0.5, -0.5, 2, -3]])
    y = pq.rms_norm(x, np.ones(4), 1e-5)
    assert np.allclose(y[0], np.array([1, 2, 3, 4]) / math.sqrt(7.5 + 1e-5), atol=1e-15)
    assert np.allclose(y[1], x[1] / math.sqrt(13.5 / 4 + 1e-5), atol=1e-15)


def test_rmsnorm_eps_is_inside_the_root_and_added_to_the_mean():
    x = rnd(3, 10, seed=8) * 1e-2
    for eps in (1e-6, 1e-2):
        y = pq.rms_norm(x, None, eps)
        ms = (x * x).mean(-1)
        assert np.allclose((y * y).mean(-1), ms / (ms + eps))     # fails for sqrt(ms)+eps and for sum+eps
    w = rnd(10, seed=9)
    assert np.allclose(pq.rms_norm(x, w, 1e-6), pq.rms_norm(x, None, 1e-6) * w)
    big = rnd(2, 10, seed=10) * 100
    assert np.allclose(pq.rms_norm(big, w, 1e-6), pq.rms_norm(3 * big, w, 1e-6), rtol=1e-8)
    lib = torch.nn.functional.rms_norm(torch.tensor(x), (10,), torch.tensor(w), 1e-6).numpy()
    assert np.allclose(pq.rms_norm(x, w, 1e-6), lib)


# ------------------------------------------------------------------ rotation
def test_rope_reference_vector():
    # src/graph/cpu_backend.rs:597-637: hd 2, 2 heads, rows at positions 0 and 1, base 10000
    x = np.array([[0.1, 0.2, 0.3, 0.4], [2.1, 2.2, 2.3, 2.4]])
    y = pq.rope_neox(x, [0, 1], 2, 2, 10000.0)
    c, s = math.cos(1.0), math.sin(1.0)
    assert np.allclose(y[0], x[0])
    assert np.allclose(y[1], [2.1 * c - 2.2 * s, 2.1 * s + 2.2 * c, 2.3 * c - 2.4 * s, 2.3 * s + 2.4 * c])


def test_rope_pairs_are_half_split_and_the_sign_is_right():
    hd = 8
    x = np.zeros((1, hd))
    x[0, 1] = 1.0
    y = pq.rope_neox(x, [3], 1, hd, 100.0)
    ang = 3.0 / 100.0 ** (2 * 1 / hd)
    assert np.nonzero(y[0])[0].tolist() == [1, 1 + hd // 2]            # not [1, 2] (interleaved) nor [0, 1]
    assert np.allclose([y[0, 1], y[0, 5]], [math.cos(ang), math.sin(ang)])   # +sin in the upper half
    # equals multiplication by e^{i angle} of (x0 + i x1)
    v = rnd(5, 3 * hd, seed=11)
    pos = [0, 1, 7, 100, 4000]
    out = pq.rope_neox(v, pos, 3, hd, 1e6).reshape(5, 3, hd)
    vh = v.reshape(5, 3, hd)
    z = (vh[..., :hd // 2] + 1j * vh[..., hd // 2:]) * np.exp(
        1j * np.array(pos)[:, None, None] / 1e6 ** (2 * np.arange(hd // 2) / hd))
    assert np.allclose(out[..., :hd // 2], z.real) and np.allclose(out[..., hd // 2:], z.imag)


# cos and sin of 1, 10, 100 and 1000 radians, from tables, not from the formula under test
COS_1_10_100_1000 = (0.5403023058681398, -0.8390715290764524, 0.8623188722876839, 0.5623790762907029)
SIN_1_10_100_1000 = (0.8414709848078965, -0.5440211108893698, -0.5063656411097588, 0.8268795405320025)


def test_rope_frequency_ladder_by_hand():
    """freq_i = theta^(-2i/hd) (src/graph/cpu_backend.rs:415, scripts/verify_rope.py:44 of
    yusiwen/minfer).  With hd 8 and theta 10^4 the four frequencies are exactly 1, 0.1, 0.01 and
    0.001, so at position 1000 the angles are 1000, 100, 10 and 1 radians: a ladder with another
    exponent (i/hd, 2i/(hd/2), (2i+1)/hd), another base or the frequencies in another order gives
    other numbers here, which no invariant of the rotation notices."""
    hd = 8
    for i in range(4):
        x = np.zeros((1, hd))
        x[0, i] = 1.0
        y = pq.rope_neox(x, [1000], 1, hd, 10000.0)[0]
        assert abs(y[i] - COS_1_10_100_1000[3 - i]) < 1e-9 and abs(y[i + 4] - SIN_1_10_100_1000[3 - i]) < 1e-9, i
    # position 1: angles 1, 0.1, 0.01, 0.001; the first pair turns by one radian exactly
    x = np.zeros((1, hd))
    x[0, 0] = 1.0
    y = pq.rope_neox(x, [1], 1, hd, 10000.0)[0]
    assert abs(y[0] - COS_1_10_100_1000[0]) < 1e-12 and abs(y[4] - SIN_1_10_100_1000[0]) < 1e-12


def test_rope_keeps_norms_and_depends_on_distance_only():
    hd = 16
    q, k = rnd(1, hd, seed=12), rnd(1, hd, seed=13)
    for m, n in ((5, 2), (105, 102), (3000, 2997)):
        qm, kn = pq.rope_neox(q, [m], 1, hd, 1e4), pq.rope_neox(k, [n], 1, hd, 1e4)
        assert np.allclose(np.linalg.norm(qm), np.linalg.norm(q))
        if m == 5:
            ref = float((qm @ kn.T)[0, 0])
        assert abs(float((qm @ kn.T)[0, 0]) - ref) < 1e-9
    assert np.allclose(pq.rope_neox(q, [0], 1, hd, 1e4), q)
    # freq_scale multiplies the frequency
    assert np.allclose(pq.rope_neox(q, [8], 1, hd, 1e4, 0.5), pq.rope_neox(q, [4], 1, hd, 1e4))


# ------------------------------------------------------------------ attention
def test_attention_reference_vector_one_key_gives_v():
    # src/graph/cpu_backend.rs:640-682: q = k = [1,0, 0,1], v = [.5,.5,.25,.75], scale .5, nh = nk = 2
    q = k = np.array([[1., 0, 0, 1]])
    v = np.array([[0.5, 0.5, 0.25, 0.75]])
    assert np.allclose(pq.gqa_attention(q, k, v, [0], [0], 2, 2, 2, 0.5), v)
    # one key, grouped heads: V is broadcast over the group (scripts/verify_attention.py:103-109)
    v2 = rnd(1, 2 * 4, seed=14)
    out = pq.gqa_attention(rnd(1, 6 * 4, seed=15), rnd(1, 2 * 4, seed=16), v2, [0], [0], 6, 2, 4, 0.3)
    assert np.allclose(out.reshape(6, 4), np.repeat(v2.reshape(2, 4), 3, axis=0))


def test_attention_equals_library_routine():
    t, nh, hd = 7, 3, 8
    q, k, v = rnd(t, nh * hd, seed=17), rnd(t, nh * hd, seed=18), rnd(t, nh * hd, seed=19)
    pos = np.arange(t)
    mine = pq.gqa_attention(q, k, v, pos, pos, nh, nh, hd, 1 / math.sqrt(hd))
    tt = lambda a: torch.tensor(a).view(t, nh, hd).transpose(0, 1)
    lib = torch.nn.functional.scaled_dot_product_attention(tt(q), tt(k), tt(v), is_causal=True)
    assert np.allclose(mine, lib.transpose(0, 1).reshape(t, nh * hd).numpy())
    # without a mask (last query sees everything): plain softmax(QK^T)V
    last = torch.nn.functional.scaled_dot_product_attention(tt(q)[:, -1:], tt(k), tt(v))
    assert np.allclose(mine[-1], last.transpose(0, 1).reshape(nh * hd).numpy())
    # grouped = repeated kv heads (h // group, not h % nk)
    nk = 1
    kg, vg = rnd(t, nk * hd, seed=20), rnd(t, nk * hd, seed=21)
    g = pq.gqa_attention(q, kg, vg, pos, pos, nh, nk, hd, 0.2)
    full = pq.gqa_attention(q, np.tile(kg, (1, nh)), np.tile(vg, (1, nh)), pos, pos, nh, nh, hd, 0.2)
    assert np.allclose(g, full)
    k2, v2 = rnd(t, 2 * hd, seed=22), rnd(t, 2 * hd, seed=23)
    g4 = pq.gqa_attention(rnd(t, 4 * hd, seed=24), k2, v2, pos, pos, 4, 2, hd, 0.2)
    rep = lambda a: np.repeat(a.reshape(t, 2, hd), 2, axis=1).reshape(t, 4 * hd)
    assert np.allclose(g4, pq.gqa_attention(rnd(t, 4 * hd, seed=24), rep(k2), rep(v2), pos, pos, 4, 4, hd, 0.2))


def test_attention_invariants():
    t, nh, nk, hd = 6, 4, 2, 4
    q, k, v = rnd(t, nh * hd, seed=25), rnd(t, nk * hd, seed=26), rnd(t, nk * hd, seed=27)
    pos = np.arange(t)
    base = pq.gqa_attention(q, k, v, pos, pos, nh, nk, hd, 0.5)
    # causal: a later token changes nothing before it
    k2, v2 = k.copy(), v.copy()
    k2[4], v2[4] = 9.0, -9.0
    other = pq.gqa_attention(q, k2, v2, pos, pos, nh, nk, hd, 0.5)
    assert np.allclose(base[:4], other[:4]) and not np.allclose(base[4:], other[4:])
    # equal scores: the mean of the visible V rows
    flat = pq.gqa_attention(q, np.zeros_like(k), v, pos, pos, nh, nk, hd, 0.5)
    assert np.allclose(flat[3].reshape(nh, hd)[0], v[:4].reshape(4, nk, hd)[:, 0].mean(0))
    # V constant per kv head: every head of the group returns it
    vc = np.tile(np.array([[1., 1, 1, 1, 2, 2, 2, 2]]), (t, 1))
    out = pq.gqa_attention(q, k, vc, pos, pos, nh, nk, hd, 0.5).reshape(t, nh, hd)
    assert np.allclose(out[:, :2], 1.0) and np.allclose(out[:, 2:], 2.0)
    # window: wide = none; 1 = own V row
    assert np.allclose(pq.gqa_attention(q, k, v, pos, pos, nh, nk, hd, 0.5, window=t), base)
    w1 = pq.gqa_attention(q, k, v, pos, pos, nh, nk, hd, 0.5, window=1).reshape(t, nh, hd)
    assert np.allclose(w1[:, 0], v.reshape(t, nk, hd)[:, 0])
    w3 = pq.gqa_attention(q, k, v, pos, pos, nh, nk, hd, 0.5, window=3)
    assert np.allclose(w3[5], pq.gqa_attention(q[5:], k[3:], v[3:], [5], [3, 4, 5], nh, nk, hd, 0.5)[0])
    # softmax shift invariance
    s = rnd(3, 5, seed=28)
    assert np.allclose(pq.softmax_rows(s), pq.softmax_rows(s + 100.0))


# ------------------------------------------------------------------ embedding, head, whole model
def test_embedding_rows_and_errors():
    e = np.array([[1., 2, 3, 4], [10, 20, 30, 40], [100, 200, 300, 400]])
    assert pq.embedding(e, [2, 0]).tolist() == [[100, 200, 300, 400], [1, 2, 3, 4]]   # cpu_backend.rs:686-709
    with pytest.raises(ValueError, match="embedding id 3 >= vocab 3"):
        pq.embedding(e, [3])


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("plain")
    return {n: pq.PlainQwen2.from_folder(write_tiny(tmp, n, seed=5)) for n in TINIES}


def test_zeroed_output_matrices_isolate_the_residual_wiring(models):
    m = models["B"]
    w = dict(m.w)
    for i in range(m.n_layers):
        w[f"model.layers.{i}.self_attn.o_proj.weight"] = np.zeros_like(w[f"model.layers.{i}.self_attn.o_proj.weight"])
        w[f"model.layers.{i}.mlp.down_proj.weight"] = np.zeros_like(w[f"model.layers.{i}.mlp.down_proj.weight"])
    z = pq.PlainQwen2(m.c, w)
    toks = random_tokens(1000, 9, 1)
    e = w["model.embed_tokens.weight"][toks]
    assert np.allclose(z.forward(toks), pq.rms_norm(e, w["model.norm.weight"], 1e-5) @ w["lm_head.weight"].T)


def test_tied_head_uses_the_embedding_table(models):
    m = models["A"]
    assert m.tied and "lm_head.weight" not in m.w
    toks = random_tokens(512, 6, 2)
    base = m.forward(toks)
    w = dict(m.w)
    w["model.embed_tokens.weight"] = w["model.embed_tokens.weight"].copy()
    w["model.embed_tokens.weight"][400] += 1.0            # a row no prompt token uses
    moved = pq.PlainQwen2(m.c, w).forward(toks)
    assert not np.allclose(base[:, 400], moved[:, 400]) and np.allclose(np.delete(base, 400, 1), np.delete(moved, 400, 1))


def test_layer_depends_on_distances_only(models):
    m = models["C"]
    h = rnd(7, 200, seed=29)
    a = m.layer(0, h, np.arange(7))
    b = m.layer(0, h, np.arange(7) + 37)
    assert np.allclose(a, b, atol=1e-9)


def test_prefix_property_and_precisions(models, tmp_path):
    m = models["A"]
    toks = random_tokens(512, 20, 3)
    full = m.forward(toks)
    assert np.allclose(full[:11], m.forward(toks[:11]), atol=1e-12)      # causal end to end
    m32 = pq.PlainQwen2(m.c, m.w, dtype=np.float32)
    assert np.abs(m32.forward(toks) - full).max() < 2e-5
    assert full.shape == (20, 512) and config_from_dict(TINIES["A"]).head_dim == m.hd == 16


# ------------------------------------------------------------------ sampling (src/sampler.rs:307-461)
def test_sampler_reference_vectors():
    f = lambda *v: np.array(v, dtype=np.float32)
    assert pq.greedy(f(1, 5, -2, 3)) == 1
    assert pq.greedy(f(2, 7, 7, 1)) == 1                               # first maximum
    assert pq.apply_penalties(f(1, 2, 3, 4), [3], 2.0, 0, 0)[3] == 2.0
    assert pq.apply_penalties(f(-4, -2, -1, -3), [3], 2.0, 0, 0)[3] == -6.0
    assert pq.apply_penalties(f(1, 2, 3), [0, 1], 1.0, 0, 0).tolist() == [1, 2, 3]
    assert pq.apply_penalties(f(1, 2, 3, 4), [3, 3], 1.0, 0.5, 0)[3] == 3.0
    assert abs(pq.apply_penalties(f(1, 2, 3, 4), [3, 3], 1.0, 0, 0.8)[3] - 3.2) < 1e-6
    assert pq.apply_penalties(f(4, -4, 0, 0), [0], 2.0, 1.0, 1.0).tolist() == [1, -4, 0, 0]
    assert pq.apply_penalties(f(4, -4, 0, 0), [1], 2.0, 0, 0).tolist() == [4, -8, 0, 0]
    assert pq.apply_penalties(f(1, 2), [99, 99], 2.0, 1.0, 1.0).tolist() == [1, 2]
    assert pq.recent_window([0, 1, 2, 3, 4, 5], 3) == [3, 4, 5] and pq.recent_window([], 64) == []
    k = pq.apply_top_k(f(1, 5, 2, 4), 2)
    assert k[1] == 5 and k[3] == 4 and np.isneginf(k[0]) and np.isneginf(k[2])
    assert pq.apply_top_k(f(1, 5, 5, 4), 1).tolist()[1:3] == [5, 5]    # ties at the threshold stay
    assert pq.apply_top_k(f(1, 2), 0).tolist() == [1, 2] and pq.apply_top_k(f(1, 2), 2).tolist() == [1, 2]
    p = pq.apply_top_p(f(1, 2, 3, 4), 0.5)
    assert np.isneginf(p[:3]).all() and p[3] == 4.0
    assert pq.apply_top_p(f(1, 2, 3, 4), 1.0).tolist() == [1, 2, 3, 4]
    assert pq.apply_top_p(f(0, 0, 0, 0), 0.3).tolist()[:2] == [0, 0]   # stable: lower indices first
    assert pq.sample(f(1, 2, 3, 4), 0.0, 0.5, 40, 0.95, 2.0, 0, 0, [3]) == 2   # greedy applies the penalty


def test_temperature_walk():
    l = np.arange(100, dtype=np.float32) * 0.1
    probs = pq.temperature_probs(l, 0.8)
    assert abs(probs.sum() - 1) < 1e-5 and np.allclose(probs, torch.softmax(torch.tensor(l) / 0.8, 0).numpy(), atol=1e-7)
    cum = np.cumsum(probs.astype(np.float64))
    for r in (0.0, 0.013, 0.5, 0.977, 0.999999):
        i = pq.sample_from_probs(probs, r)
        assert (cum[i - 1] if i else 0.0) - 1e-6 <= r <= cum[i] + 1e-6
    assert pq.sample_from_probs(probs, 0.0) == 0
    masked = pq.temperature_probs(np.array([-np.inf, 1.0, -np.inf, 1.0], dtype=np.float32), 1.0)
    assert masked.tolist() == [0, 0.5, 0, 0.5] and pq.sample_from_probs(masked, 0.0) == 1
    assert pq.sample_from_probs(masked, 0.75) == 3
    # as the temperature falls the draw converges to the argmax
    assert all(pq.sample(l, 1e-3, r) == 99 for r in (0.1, 0.5, 0.9))
    # draws follow the softmax
    rng = np.random.default_rng(0)
    small = np.array([0.0, 1.0, 2.0], dtype=np.float32)
    counts = np.bincount([pq.sample(small, 1.0, float(r)) for r in rng.random(20000)], minlength=3)
    expect = torch.softmax(torch.tensor(small), 0).numpy() * 20000
    assert (np.abs(counts - expect) < 4 * np.sqrt(expect)).all()


def test_uniform_stream():
    from minfer_amd.sampling import uniform
    u = [uniform(42, 0, s) for s in range(2000)]
    assert all(0.0 <= x < 1.0 for x in u) and abs(np.mean(u) - 0.5) < 0.03 and len(set(u)) > 1990
    assert uniform(42, 0, 5) == uniform(42, 0, 5) != uniform(42, 1, 5) != uniform(43, 0, 5)
    assert all(float(np.float32(x)) == x for x in u[:50])            # exact in float32


# ------------------------------------------------------------------ how the parts are put together
def with_random_gains(m, seed):
    """The same model with norm gains that are not one, so that where a norm stands shows."""
    w = dict(m.w)
    for n in w:
        if n.endswith("layernorm.weight") or n == "model.norm.weight":
            w[n] = 1.0 + 0.5 * rnd(*w[n].shape, seed=seed + len(n))
    return pq.PlainQwen2(m.c, w)


@pytest.mark.parametrize("name", list(TINIES))
def test_whole_model_equals_a_composition_of_library_routines(models, name):
    """The model once more, put together from torch's own routines (rms_norm, linear,
    scaled_dot_product_attention with its default scale 1/sqrt(head size) and its grouped-query
    mode, silu); only the rotation is the plain implementation's (pinned above).  Placement of
    the norms (gains are not one here), which products carry a bias (q, k, v; not o, not the
    feed-forward), the scale (TINY_C's head size is not width / heads), the head mapping and the
    tied head all have to agree.  src/models/qwen2/graph.rs:59-182."""
    F = torch.nn.functional
    m = with_random_gains(models[name], seed=31)
    c = m.c
    nh, nk = c["num_attention_heads"], c["num_key_value_heads"]
    hd = c.get("head_dim") or c["hidden_size"] // nh
    eps, theta = c["rms_norm_eps"], c["rope_theta"]
    toks = random_tokens(c["vocab_size"], 11, 7)
    t = {k: torch.tensor(v) for k, v in m.w.items()}
    n = len(toks)
    pos = np.arange(n)
    h = t["model.embed_tokens.weight"][toks]
    for i in range(c["num_hidden_layers"]):
        p = f"model.layers.{i}."
        x = F.rms_norm(h, (h.shape[-1],), t[p + "input_layernorm.weight"], eps)
        q = F.linear(x, t[p + "self_attn.q_proj.weight"], t[p + "self_attn.q_proj.bias"])
        k = F.linear(x, t[p + "self_attn.k_proj.weight"], t[p + "self_attn.k_proj.bias"])
        v = F.linear(x, t[p + "self_attn.v_proj.weight"], t[p + "self_attn.v_proj.bias"])
        q = torch.tensor(pq.rope_neox(q.numpy(), pos, nh, hd, theta)).view(n, nh, hd).transpose(0, 1)
        k = torch.tensor(pq.rope_neox(k.numpy(), pos, nk, hd, theta)).view(n, nk, hd).transpose(0, 1)
        v = v.view(n, nk, hd).transpose(0, 1)
        a = F.scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=True)      # scale: 1/sqrt(hd)
        h = h + F.linear(a.transpose(0, 1).reshape(n, nh * hd), t[p + "self_attn.o_proj.weight"])
        x = F.rms_norm(h, (h.shape[-1],), t[p + "post_attention_layernorm.weight"], eps)
        h = h + F.linear(F.silu(F.linear(x, t[p + "mlp.gate_proj.weight"])) * F.linear(x, t[p + "mlp.up_proj.weight"]),
                         t[p + "mlp.down_proj.weight"])
    x = F.rms_norm(h, (h.shape[-1],), t["model.norm.weight"], eps)
    out = F.linear(x, t["model.embed_tokens.weight"] if c.get("tie_word_embeddings") else t["lm_head.weight"])
    assert f"model.layers.0.self_attn.o_proj.bias" not in m.w and "model.layers.0.mlp.down_proj.bias" not in m.w
    assert np.abs(m.forward(toks) - out.numpy()).max() < 1e-10


def test_each_branch_reads_the_normed_stream_and_adds_to_the_raw_one(models):
    """Pre-norm: a branch sees norm(h) and its output is added to h itself.  With the other
    branch switched off (its output matrix zero), layer(c h) - c h is the same for every c > 0,
    because norm(c h) = norm(h) (eps aside); a norm after the addition, or a branch fed h itself,
    would not give that."""
    m = with_random_gains(models["B"], seed=41)
    h = rnd(6, 128, seed=42) * 3.0
    pos = np.arange(6)
    for off, what in (("mlp.down_proj.weight", "attention"), ("self_attn.o_proj.weight", "feed-forward")):
        w = dict(m.w)
        w["model.layers.0." + off] = np.zeros_like(w["model.layers.0." + off])
        z = pq.PlainQwen2(m.c, w)
        base = z.layer(0, h, pos) - h
        assert np.abs(base).max() > 1e-3, what
        for c in (0.5, 7.0):
            assert np.allclose(z.layer(0, c * h, pos) - c * h, base, rtol=1e-4, atol=1e-7), what

"""Each part alone against the plain functions, and a model put together from other parts
than the architecture's: a toy mixer with state of its own, defined here, is registered,
built and stepped without a change to the framework's files; its model runs one block
twice and lets a layer read another layer's cache."""
import math

import numpy as np
import pytest
import torch

import plain_qwen2 as pq
from minfer_amd.cache import Cache, KVRequest, StateRequest
from minfer_amd.engine.batch import StepContext
from minfer_amd.parts import (BlockSpec, ModelSpec, PartSpec, RunEntry, Runtime, Mixer, make_part, register_mixer,
                              FEED_FORWARDS, MIXERS, NORMS, POSITIONS)
from minfer_amd.weights import TensorSpec
from replays import batch_steps, compare, requests_for, run_steps, tail_steps, whole_steps

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def rnd(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


def context(cache, slots, new, start):
    """A StepContext built by hand for part-level tests."""
    n_tok = sum(new)
    seq = torch.repeat_interleave(torch.arange(len(slots)), torch.tensor(new)).int()
    pos = torch.cat([torch.arange(s, s + n) for s, n in zip(start, new)]).int()
    new_len = {s: st + n for s, st, n in zip(slots, start, new)}
    cache.reserve(new_len)
    max_len = max(new_len.values())
    cols = (max_len + 63) // 64
    tables = {id(g): torch.tensor(cache.page_rows(g, slots, cols), dtype=torch.int32, device=DEV) for g in cache.groups}
    cu = torch.tensor([0] + list(np.cumsum(new)), dtype=torch.int32)
    return StepContext(cache=cache, n_tokens=n_tok, n_seqs=len(slots), token_ids=torch.zeros(n_tok, dtype=torch.int32, device=DEV),
                       positions=pos.to(DEV), seq_of_tok=seq.to(DEV), cu_seqlens=cu.to(DEV),
                       start_pos=torch.tensor(start, dtype=torch.int32, device=DEV),
                       slot_ids=torch.tensor(slots, dtype=torch.int32, device=DEV), logit_rows=None, page_tables=tables,
                       max_len=max_len, max_new=max(new), all_decode=all(n == 1 for n in new),
                       host_new=list(new), host_start=list(start), new_lengths=new_len)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rmsnorm_part(dtype):
    rt = Runtime(dtype, DEV)
    part = make_part(NORMS, PartSpec("rmsnorm", dict(size=200, eps=3e-6, weight="n.weight")), rt, "norm")
    assert part.tensor_specs() == {"n.weight": TensorSpec((200,), init="ones")}
    w, x = rnd(200, seed=1) + 1, rnd(9, 200, seed=2, scale=4.0)
    part.load(lambda name: w.to(DEV).to(dtype))
    ref = pq.rms_norm(x.double().numpy(), w.to(dtype).double().numpy(), 3e-6)
    tol = 1e-5 if dtype == torch.float32 else 3e-2
    assert np.abs(part.forward(x.to(DEV)).float().cpu().numpy() - ref).max() < tol


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_swiglu_part_adds_into_the_residual(dtype):
    rt = Runtime(dtype, DEV)
    part = make_part(FEED_FORWARDS, PartSpec("swiglu", dict(hidden_size=72, intermediate_size=100, gate="g", up="u", down="d")), rt, "ffn")
    assert sorted(part.tensor_specs()) == ["d.weight", "g.weight", "u.weight"]
    w = {"g.weight": rnd(100, 72, seed=3, scale=0.2), "u.weight": rnd(100, 72, seed=4, scale=0.2),
         "d.weight": rnd(72, 100, seed=5, scale=0.2)}
    part.load(lambda name: w[name].to(DEV).to(dtype))
    x, h = rnd(5, 72, seed=6), rnd(5, 72, seed=7)
    hd = h.to(DEV).clone()
    part.forward(x.to(DEV).to(dtype), hd, None)
    wd = {k: v.to(dtype).double().numpy() for k, v in w.items()}
    ref = h.double().numpy() + pq.swiglu_ffn(x.to(dtype).double().numpy(), wd["g.weight"], wd["u.weight"], wd["d.weight"])
    assert np.abs(hd.cpu().numpy() - ref).max() < (1e-5 if dtype == torch.float32 else 3e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window", [None, 50])
def test_attention_part_prompt_then_decode(dtype, window):
    nh, nk, hd, hidden = 6, 2, 32, 80
    rt = Runtime(dtype, DEV)
    position = PartSpec("rope_neox", dict(head_dim=hd, theta=5000.0, max_positions=512))
    spec = PartSpec("gqa_attention", dict(hidden_size=hidden, n_heads=nh, n_kv_heads=nk, head_dim=hd, scale=0.2,
                                          window=window, qkv_bias=True, out_bias=False, position=position,
                                          q="q", k="k", v="v", o="o"))
    part = make_part(MIXERS, spec, rt, "mixer")
    assert part.cache_request() == KVRequest(nk, hd, window)
    specs = part.tensor_specs()
    assert specs["k.weight"].shape == (nk * hd, hidden) and specs["o.weight"].shape == (hidden, nh * hd) and "o.bias" not in specs
    w = {n: rnd(*s.shape, seed=10 + i, scale=0.15) for i, (n, s) in enumerate(sorted(specs.items()))}
    part.load(lambda name: w[name].to(DEV).to(dtype))
    cache = Cache({0: part.cache_request()}, 64 * 8, 4, dtype, DEV, poison=True)
    lens = [70, 130]
    slots = [cache.alloc_slot() for _ in lens]
    xs = [rnd(n, hidden, seed=20 + i) for i, n in enumerate(lens)]
    wd = {k: v.to(dtype).double().numpy() for k, v in w.items()}

    def plain(x, n):
        x = x[:n].to(dtype).double().numpy()
        pos = np.arange(n)
        q = pq.rope_neox(pq.linear(x, wd["q.weight"], wd["q.bias"]), pos, nh, hd, 5000.0)
        k = pq.rope_neox(pq.linear(x, wd["k.weight"], wd["k.bias"]), pos, nk, hd, 5000.0)
        v = pq.linear(x, wd["v.weight"], wd["v.bias"])
        return pq.linear(pq.gqa_attention(q, k, v, pos, pos, nh, nk, hd, 0.2, window), wd["o.weight"])
    tol = 2e-5 if dtype == torch.float32 else 4e-2
    # prompts (all but the last 3 tokens) in one step, then one token each
    heads = [n - 3 for n in lens]
    ctx = context(cache, slots, heads, [0, 0])
    h = torch.zeros(sum(heads), hidden, device=DEV)
    part.forward(torch.cat([x[:n] for x, n in zip(xs, heads)]).to(DEV).to(dtype), h, ctx, 0, True)
    cache.commit(ctx.new_lengths)
    ref = np.concatenate([plain(x, n) for x, n in zip(xs, heads)])
    assert np.abs(h.cpu().numpy() - ref).max() < tol
    for step in range(3):
        at = [n + step for n in heads]
        ctx = context(cache, slots, [1, 1], at)
        h = torch.zeros(2, hidden, device=DEV)
        part.forward(torch.stack([x[a] for x, a in zip(xs, at)]).to(DEV).to(dtype), h, ctx, 0, True)
        cache.commit(ctx.new_lengths)
        ref = np.stack([plain(x, a + 1)[a] for x, a in zip(xs, at)])
        assert np.abs(h.cpu().numpy() - ref).max() < tol
    cache.check_invariants()


def test_unknown_part_and_unsupported_head_size():
    rt = Runtime(torch.float32, DEV)
    with pytest.raises(KeyError, match="unknown mixer 'nope'"):
        make_part(MIXERS, PartSpec("nope", {}), rt, "mixer")
    position = PartSpec("rope_neox", dict(head_dim=24, theta=1e4, max_positions=64))
    with pytest.raises(ValueError, match="head_dim 24"):
        make_part(MIXERS, PartSpec("gqa_attention", dict(hidden_size=48, n_heads=2, n_kv_heads=2, head_dim=24, scale=1.0,
                                                         position=position, q="q", k="k", v="v", o="o")), rt, "mixer")


# ------------------------------------------------------------------ a toy architecture
DECAY = 0.75


@register_mixer("toy_decay_state")
class ToyDecayMixer(Mixer):
    """state s (one vector per sequence): s <- DECAY * s + x_t; output W s.  Written with
    torch operations on the device: a toy, not a kernel."""

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.hidden = int(spec.params["hidden_size"])
        self.w = None

    def tensor_specs(self):
        return {"toy.weight": TensorSpec((self.hidden, self.hidden))}

    def load(self, get):
        self.w = get("toy.weight").float()

    def cache_request(self):
        return StateRequest((self.hidden,), torch.float32)

    def forward(self, x, h, ctx, entry, writes_cache):
        # the sequences' rows of the state are addressed by ctx.slot_ids, on the device: which
        # slots they are is data, so a captured decode step works for any binding
        state = ctx.cache.state(entry)
        ids = ctx.slot_ids.long()
        s = state.index_select(0, ids)                    # [sequences][hidden]
        off = 0
        for b, n in enumerate(ctx.host_new):
            for t in range(off, off + n):
                s[b] = DECAY * s[b] + x[t].float()
                h[t] += self.w @ s[b]
            off += n
        state.index_copy_(0, ids, s)


class ToyConfig:
    """Layer 0: attention; layer 1: the toy mixer; run order 0, 1, 0 again (its own cache
    entry), then a second attention-only block that reads entry 0 instead of writing."""

    def __init__(self, raw):
        self.raw = raw
        self.hidden, self.vocab = raw["hidden_size"], raw["vocab_size"]

    @classmethod
    def from_dict(cls, raw):
        return cls(raw)

    def to_dict(self):
        return dict(self.raw)

    def random_init_std(self, name):
        return 0.08

    def model_spec(self):
        hid = self.hidden
        norm = lambda n: PartSpec("rmsnorm", dict(size=hid, eps=1e-5, weight=n))
        pos = PartSpec("rope_neox", dict(head_dim=16, theta=1e4, max_positions=256))
        attn = PartSpec("gqa_attention", dict(hidden_size=hid, n_heads=3, n_kv_heads=1, head_dim=16, scale=0.25, window=None,
                                              qkv_bias=False, out_bias=False, position=pos, q="a.q", k="a.k", v="a.v", o="a.o"))
        ffn = PartSpec("swiglu", dict(hidden_size=hid, intermediate_size=40, gate="f.g", up="f.u", down="f.d"))
        toy = PartSpec("toy_decay_state", dict(hidden_size=hid))
        blocks = (BlockSpec("prenorm", "l0.", attn, ffn, norm("n1"), norm("n2")),
                  BlockSpec("prenorm", "l1.", toy, ffn, norm("n1"), norm("n2")),
                  BlockSpec("prenorm", "l2.", attn, ffn, norm("n1"), norm("n2")))
        schedule = (RunEntry(0, 0), RunEntry(1, 1), RunEntry(0, 2), RunEntry(2, 0, writes_cache=False))
        return ModelSpec(hidden_size=hid, vocab_size=self.vocab, embedding_name="emb", head_name=None,
                         final_norm=norm("nf"), blocks=blocks, schedule=schedule, max_positions=256)


class PlainToy:
    """The toy model, whole sequences, numpy float64."""

    def __init__(self, folder):
        from safetensors.torch import load_file
        self.w = {k: v.double().numpy() for k, v in load_file(folder + "/model.safetensors").items()}

    def attn(self, p, x, pos, kv=None):
        w = self.w
        q = pq.rope_neox(pq.linear(x, w[p + "a.q.weight"]), pos, 3, 16, 1e4)
        if kv is None:
            kv = (pq.rope_neox(pq.linear(x, w[p + "a.k.weight"]), pos, 1, 16, 1e4), pq.linear(x, w[p + "a.v.weight"]))
        return pq.linear(pq.gqa_attention(q, kv[0], kv[1], pos, pos, 3, 1, 16, 0.25), w[p + "a.o.weight"]), kv

    def ffn(self, p, h):
        w = self.w
        return h + pq.swiglu_ffn(pq.rms_norm(h, w[p + "n2"], 1e-5), w[p + "f.g.weight"], w[p + "f.u.weight"], w[p + "f.d.weight"])

    def forward(self, tokens):
        w, pos = self.w, np.arange(len(tokens))
        h = w["emb"][tokens]
        a, kv0 = self.attn("l0.", pq.rms_norm(h, w["l0.n1"], 1e-5), pos)
        h = self.ffn("l0.", h + a)
        x, s, out = pq.rms_norm(h, w["l1.n1"], 1e-5), np.zeros(h.shape[1]), np.zeros_like(h)
        for t in range(len(tokens)):
            s = DECAY * s + x[t]
            out[t] = w["l1.toy.weight"] @ s
        h = self.ffn("l1.", h + out)
        a, _ = self.attn("l0.", pq.rms_norm(h, w["l0.n1"], 1e-5), pos)
        h = self.ffn("l0.", h + a)
        a, _ = self.attn("l2.", pq.rms_norm(h, w["l2.n1"], 1e-5), pos, kv=kv0)     # reads layer 0's keys and values
        h = self.ffn("l2.", h + a)
        return pq.rms_norm(h, w["nf"], 1e-5) @ w["emb"].T


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_architecture_is_registered_built_and_stepped(tmp_path, dtype):
    from minfer_amd import Engine, load_model, register_architecture, write_random_model
    register_architecture("ToyStateLM", ToyConfig)
    cfg = ToyConfig(dict(architectures=["ToyStateLM"], hidden_size=48, vocab_size=300))
    folder = write_random_model(str(tmp_path / "toy"), cfg, seed=3)
    model = load_model(folder, dtype=dtype)
    reqs = model.cache_requests()
    assert isinstance(reqs[1], StateRequest) and reqs[0] == reqs[2] == KVRequest(1, 16, None)
    assert "l2.a.k.weight" in model.expected_tensors()        # loaded though this entry only reads a cache
    eng = Engine(model, max_tokens=64 * 6, max_seqs=3, poison_cache=True)
    plain = PlainToy(folder)
    requests = requests_for(300, (5, 70, 33, 9), seed=4)
    ref = {r: plain.forward(t) for r, t in requests.items()}
    ids = list(requests)
    compare(run_steps(eng, whole_steps(requests)), ref, dtype, "toy whole")
    compare(run_steps(eng, tail_steps(requests, tail=8)), ref, dtype, "toy one by one")
    compare(run_steps(eng, batch_steps(requests, [ids[:3], ids[3:]])), ref, dtype, "toy batches")   # slots used again


# ------------------------------------------------------------------ more toy parts
# A feed-forward with routing, a position encoding that is not a rotation, a norm without a
# weight and a post-norm block, all defined here and put into one model: the registries, the
# loader, the cache, the step and the replays take them as they come.
from minfer_amd.parts import (Block, FeedForward, Norm, PositionEncoding, register_block,      # noqa: E402
                              register_feed_forward, register_norm, register_position)


@register_feed_forward("toy_top1_experts")
class ToyTop1Experts(FeedForward):
    """Router logits r = R x in 32-bit; the expert with the largest logit (the first on a tie)
    runs y = W2 relu(W1 x), weighted by the softmax probability of its logit."""

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        p = spec.params
        self.hidden, self.inter, self.n_experts = int(p["hidden_size"]), int(p["intermediate_size"]), int(p["experts"])

    def tensor_specs(self):
        out = {"router.weight": TensorSpec((self.n_experts, self.hidden))}
        for e in range(self.n_experts):
            out[f"e{e}.w1"] = TensorSpec((self.inter, self.hidden))
            out[f"e{e}.w2"] = TensorSpec((self.hidden, self.inter))
        return out

    def load(self, get):
        self.router = get("router.weight").float()
        self.w1 = [get(f"e{e}.w1").float() for e in range(self.n_experts)]
        self.w2 = [get(f"e{e}.w2").float() for e in range(self.n_experts)]

    def forward(self, x, h, ctx):
        x = x.float()
        logits = x @ self.router.t()
        prob = torch.softmax(logits, dim=-1)
        pick = torch.argmax(logits, dim=-1)
        for e in range(self.n_experts):
            rows = torch.nonzero(pick == e).flatten()
            if rows.numel():
                y = torch.relu(x[rows] @ self.w1[e].t()) @ self.w2[e].t()
                h[rows] += y * prob[rows, e:e + 1]


@register_position("toy_position_bias")
class ToyPositionBias(PositionEncoding):
    """No rotation: position p adds p * slope to the first element of every q and k head.  It
    treats q and k and nothing else; where keys and values go is the cache's business."""

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.head_dim, self.slope = int(spec.params["head_dim"]), float(spec.params["slope"])

    def encode(self, qkv, ctx, n_heads, n_kv_heads):
        x = qkv.view(qkv.shape[0], n_heads + 2 * n_kv_heads, self.head_dim)
        x[:, :n_heads + n_kv_heads, 0] += (ctx.positions.float() * self.slope)[:, None]


@register_norm("toy_scale_norm")
class ToyScaleNorm(Norm):
    """y = x / (mean |x| + eps): no weight, not an RMS norm, so nothing folds it into a product."""

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.eps = float(spec.params["eps"])

    def forward(self, h, out=None, row_idx=None):
        src = h if row_idx is None else h[row_idx.long()]
        y = (src / (src.abs().mean(dim=-1, keepdim=True) + self.eps)).to(self.rt.dtype)
        if out is not None:
            out.copy_(y)
            return out
        return y


@register_block("toy_postnorm")
class ToyPostNormBlock(Block):
    """h <- norm1(h + mixer(h)); h <- norm2(h + feed_forward(h)): the parts get the residual
    stream itself as their input."""

    def forward(self, h, ctx, entry, writes_cache, keep_rows=None):
        self.mixer.forward(h.to(self.rt.dtype), h, ctx, entry, writes_cache)
        h.copy_(self.mixer_norm.forward(h).float())
        if keep_rows is not None:
            h = h[keep_rows.long()].contiguous()
        self.feed_forward.forward(h.to(self.rt.dtype), h, ctx)
        h.copy_(self.feed_forward_norm.forward(h).float())
        return h


class ToyRoutedConfig(ToyConfig):
    def model_spec(self):
        hid = self.hidden
        snorm = lambda: PartSpec("toy_scale_norm", dict(eps=1e-3))
        pos = PartSpec("toy_position_bias", dict(head_dim=16, slope=0.01))
        attn = PartSpec("gqa_attention", dict(hidden_size=hid, n_heads=4, n_kv_heads=2, head_dim=16, scale=0.25, window=None,
                                              qkv_bias=True, out_bias=False, position=pos, q="a.q", k="a.k", v="a.v", o="a.o"))
        moe = PartSpec("toy_top1_experts", dict(hidden_size=hid, intermediate_size=24, experts=3))
        blocks = (BlockSpec("toy_postnorm", "l0.", attn, moe, snorm(), snorm()),
                  BlockSpec("toy_postnorm", "l1.", attn, moe, snorm(), snorm()))
        return ModelSpec(hidden_size=hid, vocab_size=self.vocab, embedding_name="emb", head_name="head",
                         final_norm=PartSpec("rmsnorm", dict(size=hid, eps=1e-5, weight="nf")), blocks=blocks,
                         schedule=(RunEntry(0, 0), RunEntry(1, 1)), max_positions=256)


class PlainRouted:
    def __init__(self, folder):
        from safetensors.torch import load_file
        self.w = {k: v.double().numpy() for k, v in load_file(folder + "/model.safetensors").items()}

    @staticmethod
    def snorm(h):
        return h / (np.abs(h).mean(axis=-1, keepdims=True) + 1e-3)

    def forward(self, tokens):
        w, pos = self.w, np.arange(len(tokens))
        h = w["emb"][tokens]
        for p in ("l0.", "l1."):
            q = pq.linear(h, w[p + "a.q.weight"], w[p + "a.q.bias"]).reshape(len(tokens), 4, 16)
            k = pq.linear(h, w[p + "a.k.weight"], w[p + "a.k.bias"]).reshape(len(tokens), 2, 16)
            v = pq.linear(h, w[p + "a.v.weight"], w[p + "a.v.bias"])
            q[:, :, 0] += pos[:, None] * 0.01
            k[:, :, 0] += pos[:, None] * 0.01
            a = pq.gqa_attention(q.reshape(len(tokens), -1), k.reshape(len(tokens), -1), v, pos, pos, 4, 2, 16, 0.25)
            h = self.snorm(h + pq.linear(a, w[p + "a.o.weight"]))
            logits = h @ w[p + "router.weight"].T
            prob = np.exp(logits - logits.max(axis=-1, keepdims=True))
            prob /= prob.sum(axis=-1, keepdims=True)
            out = np.zeros_like(h)
            for t in range(len(tokens)):
                e = int(np.argmax(logits[t]))
                out[t] = (w[p + f"e{e}.w2"] @ np.maximum(w[p + f"e{e}.w1"] @ h[t], 0.0)) * prob[t, e]
            h = self.snorm(h + out)
        return pq.rms_norm(h, w["nf"], 1e-5) @ w["head"].T


def test_toy_routing_position_norm_and_block_parts(tmp_path):
    """32-bit only: a routing decision is a jump, and bfloat16 rounding would move tokens that
    sit on one across it; the architecture's own bfloat16 runs are covered elsewhere."""
    from minfer_amd import Engine, load_model, register_architecture, write_random_model
    register_architecture("ToyRoutedLM", ToyRoutedConfig)
    cfg = ToyRoutedConfig(dict(architectures=["ToyRoutedLM"], hidden_size=40, vocab_size=211))
    folder = write_random_model(str(tmp_path / "routed"), cfg, seed=5)
    model = load_model(folder, dtype="float32")
    assert "l1.e2.w2" in model.expected_tensors() and "l0.router.weight" in model.expected_tensors()
    eng = Engine(model, max_tokens=64 * 6, max_seqs=3, poison_cache=True)
    plain = PlainRouted(folder)
    requests = requests_for(211, (6, 67, 30, 11), seed=6)
    ref = {r: plain.forward(t) for r, t in requests.items()}
    picks = [int(np.argmax(plain.w["emb"][t] @ plain.w["l0.router.weight"].T, axis=-1).max()) for t in requests.values()]
    assert max(picks) >= 1, "the routing is exercised: not every token goes to expert 0"
    ids = list(requests)
    compare(run_steps(eng, whole_steps(requests)), ref, "float32", "routed whole")
    compare(run_steps(eng, tail_steps(requests, tail=8)), ref, "float32", "routed one by one")
    compare(run_steps(eng, batch_steps(requests, [ids[:3], ids[3:]])), ref, "float32", "routed batches")


# ------------------------------------------------------------------ the toy state through the captured decode step
@pytest.mark.parametrize("dtype", ["float32"])
def test_toy_state_mixer_through_generate_with_a_captured_step(tmp_path, dtype):
    """Two batches through `generate(use_graph=True)`: the second finds its sequences in other
    slots than the ones the decode step was captured with.  Per-sequence state is addressed
    through `ctx.slot_ids` only, so the replayed step reads and writes the right rows; greedy
    tokens equal the plain model's."""
    from minfer_amd import Engine, generate, load_model, register_architecture, write_random_model
    from minfer_amd.sampling import SamplingParams
    register_architecture("ToyStateLM", ToyConfig)
    cfg = ToyConfig(dict(architectures=["ToyStateLM"], hidden_size=48, vocab_size=300))
    folder = write_random_model(str(tmp_path / "toy"), cfg, seed=7)
    eng = Engine(load_model(folder, dtype=dtype), max_tokens=64 * 8, max_seqs=5, poison_cache=True)
    plain = PlainToy(folder)
    prompts = [[int(t) for t in np.random.default_rng(40 + i).integers(0, 300, size=n)] for i, n in enumerate((4, 7, 5, 6))]

    def expected(p, n):
        seq, out = list(p), []
        for _ in range(n):
            out.append(pq.greedy(plain.forward(seq)[-1].astype(np.float32)))
            seq.append(out[-1])
        return out
    want = [expected(p, 6) for p in prompts]
    first = generate(eng, prompts[:2], SamplingParams.greedy(), max_new=6, stop_tokens=[], use_graph=True)
    assert first.tokens == want[:2]
    sessions = dict(eng._sessions)
    assert len(sessions) == 1 and next(iter(sessions.values())).graph is not None
    used = set(next(iter(sessions.values())).slots)
    blockers = [eng.new_sequence() for _ in range(2)]              # take the slots that were just given back
    second = generate(eng, prompts[2:], SamplingParams.greedy(), max_new=6, stop_tokens=[], use_graph=True)
    session = next(iter(eng._sessions.values()))
    assert dict(eng._sessions).keys() == sessions.keys(), "the same captured step served both batches"
    assert set(session.slots) != used, "the second batch lives in other slots"
    assert second.tokens == want[2:]
    for s in blockers:
        eng.end_sequence(s)
    assert not eng.cache.live_slots()


# ------------------------------------------------------------------ other ends of the model
from minfer_amd.parts import Embedding, Head, register_embedding, register_head      # noqa: E402


@register_embedding("toy_scaled_embedding")
class ToyScaledEmbedding(Embedding):
    """Rows of the table times a constant."""

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.vocab, self.hidden, self.scale = int(spec.params["vocab_size"]), int(spec.params["hidden_size"]), float(spec.params["scale"])

    def tensor_specs(self):
        return {"emb": TensorSpec((self.vocab, self.hidden))}

    def load(self, get):
        self.weight = get("emb").float()

    def table(self):
        return self.weight

    def forward(self, token_ids, out, ctx):
        out.copy_(self.weight[token_ids.long()] * self.scale)


@register_head("toy_capped_head")
class ToyCappedHead(Head):
    """logits = cap * tanh((W x + b) / cap), W tied to the embedding table."""

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.vocab, self.cap = int(spec.params["vocab_size"]), float(spec.params["cap"])

    def tensor_specs(self):
        return {"head_bias": TensorSpec((self.vocab,))}

    def load(self, get):
        self.bias = get("head_bias").float()

    def tie(self, embedding):
        self.w = embedding.table()

    def forward(self, x, ctx):
        return (self.cap * torch.tanh((x.float() @ self.w.t() + self.bias) / self.cap)).contiguous()


class ToyEndsConfig(ToyConfig):
    def model_spec(self):
        hid = self.hidden
        norm = lambda n: PartSpec("rmsnorm", dict(size=hid, eps=1e-5, weight=n))
        pos = PartSpec("rope_neox", dict(head_dim=16, theta=1e4, max_positions=256))
        attn = PartSpec("gqa_attention", dict(hidden_size=hid, n_heads=2, n_kv_heads=2, head_dim=16, scale=0.25, window=None,
                                              qkv_bias=False, out_bias=False, position=pos, q="a.q", k="a.k", v="a.v", o="a.o"))
        ffn = PartSpec("swiglu", dict(hidden_size=hid, intermediate_size=40, gate="f.g", up="f.u", down="f.d"))
        sizes = dict(vocab_size=self.vocab, hidden_size=hid)
        return ModelSpec(hidden_size=hid, vocab_size=self.vocab, final_norm=norm("nf"),
                         blocks=(BlockSpec("prenorm", "l0.", attn, ffn, norm("n1"), norm("n2")),),
                         schedule=(RunEntry(0, 0),), max_positions=256,
                         embedding=PartSpec("toy_scaled_embedding", dict(sizes, scale=3.0)),
                         head=PartSpec("toy_capped_head", dict(sizes, cap=0.5)))


def test_other_embedding_and_head_parts_without_touching_the_model(tmp_path):
    """A scaled embedding and a capped, biased, tied head are registered parts; the model's step
    is the same code."""
    from minfer_amd import Engine, load_model, register_architecture, write_random_model
    from safetensors.torch import load_file
    register_architecture("ToyEndsLM", ToyEndsConfig)
    cfg = ToyEndsConfig(dict(architectures=["ToyEndsLM"], hidden_size=32, vocab_size=150))
    folder = write_random_model(str(tmp_path / "ends"), cfg, seed=9)
    model = load_model(folder, dtype="float32")
    assert set(model.expected_tensors()) >= {"emb", "head_bias", "nf"} and "lm_head.weight" not in model.expected_tensors()
    w = {k: v.double().numpy() for k, v in load_file(folder + "/model.safetensors").items()}

    def plain(tokens):
        pos = np.arange(len(tokens))
        h = w["emb"][tokens] * 3.0
        x = pq.rms_norm(h, w["l0.n1"], 1e-5)
        q = pq.rope_neox(pq.linear(x, w["l0.a.q.weight"]), pos, 2, 16, 1e4)
        k = pq.rope_neox(pq.linear(x, w["l0.a.k.weight"]), pos, 2, 16, 1e4)
        a = pq.gqa_attention(q, k, pq.linear(x, w["l0.a.v.weight"]), pos, pos, 2, 2, 16, 0.25)
        h = h + pq.linear(a, w["l0.a.o.weight"])
        h = h + pq.swiglu_ffn(pq.rms_norm(h, w["l0.n2"], 1e-5), w["l0.f.g.weight"], w["l0.f.u.weight"], w["l0.f.d.weight"])
        return 0.5 * np.tanh((pq.rms_norm(h, w["nf"], 1e-5) @ w["emb"].T + w["head_bias"]) / 0.5)
    eng = Engine(model, max_tokens=64 * 4, max_seqs=2, poison_cache=True)
    requests = requests_for(150, (9, 70), seed=2)
    ref = {r: plain(t) for r, t in requests.items()}
    compare(run_steps(eng, whole_steps(requests)), ref, "float32", "toy ends whole")
    compare(run_steps(eng, tail_steps(requests, tail=5)), ref, "float32", "toy ends one by one")


# ------------------------------------------------------------------ other arrangements, and ends that know the positions
@register_block("toy_sandwich")
class ToySandwichBlock(Block):
    """Four norms: h += post(mixer(pre(h))); h += post(feed_forward(pre(h))).  The branch's output
    is collected in a buffer of its own, normed, and only then added to the stream."""

    norm_names = ("mixer", "mixer_post", "feed_forward", "feed_forward_post")

    def forward(self, h, ctx, entry, writes_cache, keep_rows=None):
        branch = torch.zeros_like(h)
        self.mixer.forward(self.norms["mixer"].forward(h), branch, ctx, entry, writes_cache)
        h += self.norms["mixer_post"].forward(branch).float()
        if keep_rows is not None:
            h = h[keep_rows.long()].contiguous()
        branch = torch.zeros_like(h)
        self.feed_forward.forward(self.norms["feed_forward"].forward(h), branch, ctx)
        h += self.norms["feed_forward_post"].forward(branch).float()
        return h


@register_embedding("toy_positional_embedding")
class ToyPositionalEmbedding(Embedding):
    """Learned absolute positions: row of the token table plus row of a position table, which
    only the step's context can tell."""

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.vocab, self.hidden, self.n_pos = (int(spec.params[k]) for k in ("vocab_size", "hidden_size", "positions"))

    def tensor_specs(self):
        return {"emb": TensorSpec((self.vocab, self.hidden)), "pos_emb": TensorSpec((self.n_pos, self.hidden))}

    def load(self, get):
        self.weight, self.pos = get("emb").float(), get("pos_emb").float()

    def forward(self, token_ids, out, ctx):
        out.copy_(self.weight[token_ids.long()] + self.pos[ctx.positions.long()])


@register_head("toy_position_head")
class ToyPositionHead(Head):
    """logits = W x + slope * (position of the row): the head asks the context which rows it got."""

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.vocab, self.hidden, self.slope = int(spec.params["vocab_size"]), int(spec.params["hidden_size"]), float(spec.params["slope"])

    def tensor_specs(self):
        return {"head": TensorSpec((self.vocab, self.hidden))}

    def load(self, get):
        self.w = get("head").float()

    def forward(self, x, ctx):
        pos = ctx.positions if ctx.logit_rows is None else ctx.positions[ctx.logit_rows.long()]
        return (x.float() @ self.w.t() + self.slope * pos.float()[:, None]).contiguous()


class ToySandwichConfig(ToyConfig):
    """Block 0: four norms around attention and SwiGLU.  Block 1: a pre-norm block that has a mixer
    and no feed-forward.  Block 2: a pre-norm block that has a feed-forward and no mixer."""

    def model_spec(self):
        hid = self.hidden
        norm = lambda n: PartSpec("rmsnorm", dict(size=hid, eps=1e-5, weight=n))
        pos = PartSpec("rope_neox", dict(head_dim=16, theta=1e4, max_positions=256))
        attn = PartSpec("gqa_attention", dict(hidden_size=hid, n_heads=4, n_kv_heads=2, head_dim=16, scale=0.25, window=None,
                                              qkv_bias=True, out_bias=False, position=pos, q="a.q", k="a.k", v="a.v", o="a.o"))
        ffn = PartSpec("swiglu", dict(hidden_size=hid, intermediate_size=72, gate="f.g", up="f.u", down="f.d"))
        sizes = dict(vocab_size=self.vocab, hidden_size=hid)
        blocks = (BlockSpec("toy_sandwich", "l0.", attn, ffn, norms={"mixer": norm("n1"), "mixer_post": norm("n2"),
                                                                     "feed_forward": norm("n3"), "feed_forward_post": norm("n4")}),
                  BlockSpec("prenorm", "l1.", mixer=attn, mixer_norm=norm("n1")),
                  BlockSpec("prenorm", "l2.", feed_forward=ffn, feed_forward_norm=norm("n2")))
        return ModelSpec(hidden_size=hid, vocab_size=self.vocab, final_norm=norm("nf"), blocks=blocks,
                         schedule=(RunEntry(0, 0), RunEntry(1, 1), RunEntry(2, 2)), max_positions=256,
                         embedding=PartSpec("toy_positional_embedding", dict(sizes, positions=256)),
                         head=PartSpec("toy_position_head", dict(sizes, slope=0.002)))

    def random_init_std(self, name):
        return 0.3 if name in ("emb", "pos_emb") else 0.08


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_four_norm_block_blocks_without_a_branch_and_ends_that_see_positions(tmp_path, dtype):
    """Registered from here alone: a block of four norms, pre-norm blocks that lack a feed-forward
    or a mixer, an embedding with learned absolute positions and a head that adds a term of the
    row's position (both get the step's context).  Whole, one by one and in unequal batches
    against a plain version written out below."""
    from minfer_amd import Engine, load_model, register_architecture, write_random_model
    from safetensors.torch import load_file
    register_architecture("ToySandwichLM", ToySandwichConfig)
    cfg = ToySandwichConfig(dict(architectures=["ToySandwichLM"], hidden_size=64, vocab_size=190))
    folder = write_random_model(str(tmp_path / "sandwich"), cfg, seed=13)
    model = load_model(folder, dtype=dtype)
    names = set(model.expected_tensors())
    assert {"l0.n4", "l1.n1", "l2.n2", "pos_emb", "head"} <= names and "l1.n2" not in names and "l1.f.g.weight" not in names
    assert "l2.a.q.weight" not in names
    assert model.blocks[1].feed_forward is None and model.blocks[2].mixer is None
    assert model.cache_requests()[2] is None and isinstance(model.cache_requests()[1], KVRequest)
    w = {k: v.double().numpy() for k, v in load_file(folder + "/model.safetensors").items()}

    def attention(p, x, pos):
        q = pq.rope_neox(pq.linear(x, w[p + "a.q.weight"], w[p + "a.q.bias"]), pos, 4, 16, 1e4)
        k = pq.rope_neox(pq.linear(x, w[p + "a.k.weight"], w[p + "a.k.bias"]), pos, 2, 16, 1e4)
        a = pq.gqa_attention(q, k, pq.linear(x, w[p + "a.v.weight"], w[p + "a.v.bias"]), pos, pos, 4, 2, 16, 0.25)
        return pq.linear(a, w[p + "a.o.weight"])

    def ffn(p, x):
        return pq.swiglu_ffn(x, w[p + "f.g.weight"], w[p + "f.u.weight"], w[p + "f.d.weight"])

    def plain(tokens):
        pos = np.arange(len(tokens))
        n = lambda x, name: pq.rms_norm(x, w[name], 1e-5)
        h = w["emb"][tokens] + w["pos_emb"][pos]
        h = h + n(attention("l0.", n(h, "l0.n1"), pos), "l0.n2")
        h = h + n(ffn("l0.", n(h, "l0.n3")), "l0.n4")
        h = h + attention("l1.", n(h, "l1.n1"), pos)
        h = h + ffn("l2.", n(h, "l2.n2"))
        return n(h, "nf") @ w["head"].T + 0.002 * pos[:, None]
    eng = Engine(model, max_tokens=64 * 6, max_seqs=3, poison_cache=True)
    requests = requests_for(190, (9, 70, 3, 31), seed=4)
    ref = {r: plain(t) for r, t in requests.items()}
    ids = list(requests)
    compare(run_steps(eng, whole_steps(requests)), ref, dtype, "sandwich whole", layers=3)
    compare(run_steps(eng, tail_steps(requests, tail=6)), ref, dtype, "sandwich one by one", layers=3)
    compare(run_steps(eng, batch_steps(requests, [ids[:3], ids[3:]])), ref, dtype, "sandwich batches", layers=3)
    # "last" rows only: the head is told which rows it got
    s = eng.new_sequence()
    last = eng.step([s], [requests["r1"]], "last").cpu().numpy()
    eng.end_sequence(s)
    tol = 1e-4 if dtype == "float32" else 0.055 * 2 * float(ref["r1"][-1].std())
    assert np.abs(last[0] - ref["r1"][-1]).max() < tol


def test_block_specs_are_checked_against_their_arrangement():
    """A spec that leaves out a norm its arrangement needs, names one it does not know, or lacks
    the mixer of an arrangement that needs one is refused with the block's name."""
    from minfer_amd.engine.model import _build_block
    rt = Runtime(torch.float32, torch.device("cpu"))
    norm = lambda n: PartSpec("rmsnorm", dict(size=8, eps=1e-5, weight=n))
    ffn = PartSpec("swiglu", dict(hidden_size=8, intermediate_size=8, gate="g", up="u", down="d"))
    with pytest.raises(ValueError, match="l7.*norms missing.*mixer_post"):
        _build_block(BlockSpec("toy_sandwich", "l7.", ffn, ffn, norms={"mixer": norm("a"), "feed_forward": norm("b"),
                                                                      "feed_forward_post": norm("c")}), rt)
    with pytest.raises(ValueError, match="not known to the arrangement \\['extra'\\]"):
        _build_block(BlockSpec("prenorm", "l0.", feed_forward=ffn, feed_forward_norm=norm("b"), norms={"extra": norm("x")}), rt)
    with pytest.raises(ValueError, match="needs a mixer"):
        _build_block(BlockSpec("toy_sandwich", "l1.", None, ffn), rt)
    with pytest.raises(ValueError, match="come together"):
        _build_block(BlockSpec("prenorm", "l2.", feed_forward=ffn), rt)
    with pytest.raises(ValueError, match="given twice"):
        BlockSpec("prenorm", "l3.", feed_forward=ffn, feed_forward_norm=norm("a"), norms={"feed_forward": norm("b")})

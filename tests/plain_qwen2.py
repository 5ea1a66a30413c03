"""Plain, slow implementation of the Qwen2 dense decoder, written from the formulas of
yusiwen/minfer (paths below are relative to that repository).

Whole sequences, no cache, numpy only, one function per part.  It shares no code with
``minfer_amd``: it has its own safetensors reading (through the ``safetensors`` library),
its own rotation angles, its own attention.  Arithmetic is float64 by default, a superset
of the accumulator widths the reference uses (f64 sums in ``src/vec_ops.rs:31-35,190-196,
442-446``), so the result does not depend on summation order to the precision the tests
ask for.
"""
from __future__ import annotations

import json
import math
import os

import numpy as np


# --------------------------------------------------------------------------- parts

def embedding(table: np.ndarray, ids) -> np.ndarray:
    """Row copy, no scaling; an id outside the table is an error.
    src/graph/builder.rs:60-76, src/graph/cpu_backend.rs:269-285."""
    ids = np.asarray(ids, dtype=np.int64)
    if ids.size and (ids.min() < 0 or ids.max() >= table.shape[0]):
        raise ValueError(f"embedding id {int(ids.max())} >= vocab {table.shape[0]}")
    return table[ids].copy()


def rms_norm(x: np.ndarray, w, eps: float) -> np.ndarray:
    """y = x * 1/sqrt(mean(x^2) + eps) * w, eps inside the root, added to the mean.
    src/vec_ops.rs:500-522 (weighted), :430-453 (w absent)."""
    ms = np.mean(x * x, axis=-1, keepdims=True)
    y = x * (1.0 / np.sqrt(ms + eps))
    return y if w is None else y * w


def linear(x: np.ndarray, w: np.ndarray, b=None) -> np.ndarray:
    """out[t][o] = dot(W[o][:], x[t][:]) (+ b[o]); W is [out][in].
    src/graph/cpu_backend.rs:214-248, layout src/graph/builder.rs:94-99."""
    y = x @ w.T
    return y if b is None else y + b


def rope_neox(x: np.ndarray, positions, n_heads: int, head_dim: int, theta: float,
              freq_scale: float = 1.0) -> np.ndarray:
    """Half-split ("NeoX", non-interleaved) rotation over the whole head:
    freq_i = freq_scale / theta^(2i/hd); angle = pos*freq_i; pair (i, i+hd/2);
    x0' = x0*cos - x1*sin, x1' = x0*sin + x1*cos.
    src/graph/cpu_backend.rs:403-434 (style NonInterleaved, src/models/qwen2/loader.rs:144)."""
    t = x.shape[0]
    half = head_dim // 2
    xh = x.reshape(t, n_heads, head_dim)
    i = np.arange(half, dtype=np.float64)
    freq = freq_scale / np.power(float(theta), 2.0 * i / head_dim)
    ang = np.asarray(positions, dtype=np.float64)[:, None] * freq[None, :]
    cs, sn = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
    x0, x1 = xh[..., :half], xh[..., half:]
    out = np.concatenate([x0 * cs - x1 * sn, x0 * sn + x1 * cs], axis=-1)
    return out.reshape(t, n_heads * head_dim).astype(x.dtype)


def softmax_rows(s: np.ndarray) -> np.ndarray:
    """exp(s - max) / sum; masked entries are -inf and contribute 0.
    src/vec_ops.rs:179-197, src/graph/cpu_backend.rs:470-478."""
    m = np.max(s, axis=-1, keepdims=True)
    e = np.exp(s - m)
    return e / np.sum(e, axis=-1, keepdims=True)


def gqa_attention(q: np.ndarray, k: np.ndarray, v: np.ndarray, positions_q, positions_k,
                  n_heads: int, n_kv_heads: int, head_dim: int, scale: float,
                  window=None) -> np.ndarray:
    """Grouped-query causal attention.  Query head h reads kv head h // (nh/nk); a query at
    position p sees keys at positions 0..p (src/graph/cpu_backend.rs:437-494, vl = pos+1 at
    :462).  ``window`` (absent in the reference, which has no such layer) keeps only the
    last ``window`` of those keys: p - window < j <= p."""
    tq, tk = q.shape[0], k.shape[0]
    g = n_heads // n_kv_heads
    qh = q.reshape(tq, n_heads, head_dim)
    kh = k.reshape(tk, n_kv_heads, head_dim)
    vh = v.reshape(tk, n_kv_heads, head_dim)
    pq = np.asarray(positions_q)[:, None]
    pk = np.asarray(positions_k)[None, :]
    visible = pk <= pq
    if window is not None:
        visible &= pk > pq - window
    out = np.zeros_like(qh)
    for h in range(n_heads):
        hk = h // g
        s = (qh[:, h, :] @ kh[:, hk, :].T) * scale
        s = np.where(visible, s, -np.inf)
        out[:, h, :] = softmax_rows(s) @ vh[:, hk, :]
    return out.reshape(tq, n_heads * head_dim)


def silu(z: np.ndarray) -> np.ndarray:
    """z / (1 + exp(-z)).  src/vec_ops.rs:131-146."""
    return z / (1.0 + np.exp(-z))


def swiglu_ffn(x: np.ndarray, w_gate, w_up, w_down) -> np.ndarray:
    """down( silu(gate x) * (up x) ), no biases.
    src/models/qwen2/graph.rs:170-174, src/graph/cpu_backend.rs:323-329."""
    return linear(silu(linear(x, w_gate)) * linear(x, w_up), w_down)


# --------------------------------------------------------------------------- model

class StreamedWeights:
    """Tensors of one safetensors file by name, each read (and widened) when it is asked for and
    not kept."""

    def __init__(self, path: str, dtype=np.float64):
        from safetensors import safe_open
        self._file = safe_open(path, framework="pt")
        self._names = set(self._file.keys())
        self._dtype = dtype

    def __contains__(self, name: str) -> bool:
        return name in self._names

    def __getitem__(self, name: str) -> np.ndarray:
        import torch
        return self._file.get_tensor(name).to(torch.float64).numpy().astype(self._dtype, copy=False)

    def get(self, name: str, default=None):
        return self[name] if name in self._names else default


class _LayerWeights(dict):
    """One layer's tensors, read once on first use and kept while the layer runs."""

    def __init__(self, source, prefix: str):
        super().__init__()
        self._source, self._prefix = source, prefix

    def __missing__(self, name: str):
        self[name] = self._source[name]
        return self[name]

    def get(self, name: str, default=None):
        if name in self:
            return self[name]
        v = self._source.get(name, default)
        if v is not None:
            self[name] = v
        return v

class PlainQwen2:
    """Weights as float64 arrays by their names in the file, hyper-parameters by their
    config.json keys.  ``forward`` runs one whole sequence from position 0."""

    def __init__(self, config: dict, weights: dict, dtype=np.float64):
        self.c = dict(config)
        self.w = {k: np.asarray(v, dtype=dtype) for k, v in weights.items()}
        self.dtype = dtype
        c = self.c
        self.nh = int(c["num_attention_heads"])
        self.nk = int(c.get("num_key_value_heads") or self.nh)
        self.hd = int(c.get("head_dim") or c["hidden_size"] // self.nh)
        self.eps = float(c.get("rms_norm_eps", 1e-6))
        self.theta = float(c.get("rope_theta", 10000.0))
        self.n_layers = int(c["num_hidden_layers"])
        self.tied = bool(c.get("tie_word_embeddings", False))

    @classmethod
    def from_folder(cls, folder: str, dtype=np.float64, streamed: bool = False) -> "PlainQwen2":
        """`streamed`: tensors are read from the file each time they are used instead of all at
        once, so a model of many gigabytes takes the host memory of one tensor at a time (run such
        a model with `forward_many`, which reads every layer once for all requests)."""
        import torch
        from safetensors.torch import load_file
        with open(os.path.join(folder, "config.json")) as f:
            config = json.load(f)
        path = os.path.join(folder, "model.safetensors")
        if streamed:
            model = cls(config, {}, dtype)
            model.w = StreamedWeights(path, dtype)
            return model
        raw = load_file(path)
        weights = {k: t.to(torch.float64).numpy() for k, t in raw.items()}
        return cls(config, weights, dtype)

    def layer(self, i: int, h: np.ndarray, positions, w=None) -> np.ndarray:
        """norm -> QKV(+bias) -> rope(q,k) -> attention -> O -> add -> norm -> SwiGLU -> add.
        src/models/qwen2/graph.rs:59-177; scale 1/sqrt(hd) src/models/qwen2/loader.rs:36-38.
        `w`: the layer's tensors if the caller holds them already (`forward_many`)."""
        w, p = self.w if w is None else w, f"model.layers.{i}."
        xn = rms_norm(h, w[p + "input_layernorm.weight"], self.eps)
        q = linear(xn, w[p + "self_attn.q_proj.weight"], w.get(p + "self_attn.q_proj.bias"))
        k = linear(xn, w[p + "self_attn.k_proj.weight"], w.get(p + "self_attn.k_proj.bias"))
        v = linear(xn, w[p + "self_attn.v_proj.weight"], w.get(p + "self_attn.v_proj.bias"))
        q = rope_neox(q, positions, self.nh, self.hd, self.theta)
        k = rope_neox(k, positions, self.nk, self.hd, self.theta)
        a = gqa_attention(q, k, v, positions, positions, self.nh, self.nk, self.hd,
                          1.0 / math.sqrt(self.hd))
        h = h + linear(a, w[p + "self_attn.o_proj.weight"])
        xn = rms_norm(h, w[p + "post_attention_layernorm.weight"], self.eps)
        h = h + swiglu_ffn(xn, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"],
                           w[p + "mlp.down_proj.weight"])
        return h

    def hidden(self, tokens) -> np.ndarray:
        positions = np.arange(len(tokens))
        h = embedding(self.w["model.embed_tokens.weight"], tokens)
        for i in range(self.n_layers):
            h = self.layer(i, h, positions)
        return h

    def head(self, h: np.ndarray) -> np.ndarray:
        """Final norm, then the output matrix, which is the embedding table when tied.
        src/models/qwen2/graph.rs:180-182, tie src/models/qwen2/loader.rs:260."""
        xn = rms_norm(h, self.w["model.norm.weight"], self.eps)
        wout = self.w["model.embed_tokens.weight"] if self.tied else self.w["lm_head.weight"]
        return linear(xn, wout)

    def forward(self, tokens) -> np.ndarray:
        """Logits [len(tokens), vocab] for one sequence starting at position 0."""
        return self.head(self.hidden(tokens))

    def forward_many(self, requests: dict) -> dict:
        """`forward` for every request of {id: tokens}, layer by layer over all of them, so that
        streamed weights are read once.  The requests do not see each other."""
        hs = {r: embedding(self.w["model.embed_tokens.weight"], toks) for r, toks in requests.items()}
        for i in range(self.n_layers):
            layer = _LayerWeights(self.w, f"model.layers.{i}.")
            for r, toks in requests.items():
                hs[r] = self.layer(i, hs[r], np.arange(len(toks)), layer)
        xs = {r: rms_norm(h, self.w["model.norm.weight"], self.eps) for r, h in hs.items()}
        wout = self.w["model.embed_tokens.weight"] if self.tied else self.w["lm_head.weight"]
        return {r: linear(x, wout) for r, x in xs.items()}


# --------------------------------------------------------------------------- sampling

def greedy(logits: np.ndarray) -> int:
    """First maximum under strict '>' (lowest index wins ties).  src/sampler.rs:16-26."""
    best, best_v = 0, logits[0]
    for i, v in enumerate(logits):
        if v > best_v:
            best, best_v = i, v
    return best


def apply_penalties(logits: np.ndarray, prev_tokens, repeat: float, frequency: float,
                    presence: float) -> np.ndarray:
    """Per distinct token of the window with count c: l -= c*frequency; l -= presence;
    then, if repeat >= 1 and != 1: l = l*repeat if l <= 0 else l/repeat.
    src/sampler.rs:44-76."""
    out = np.array(logits, dtype=np.float32)
    if abs(repeat - 1.0) < 1e-6 and abs(frequency) < 1e-6 and abs(presence) < 1e-6:
        return out
    counts: dict = {}
    for t in prev_tokens:
        counts[int(t)] = counts.get(int(t), 0) + 1
    for t, c in counts.items():
        if t >= len(out):
            continue
        v = np.float32(out[t])
        if abs(frequency) >= 1e-6 or abs(presence) >= 1e-6:
            v = np.float32(v - np.float32(c) * np.float32(frequency))
            v = np.float32(v - np.float32(presence))
        if abs(repeat - 1.0) >= 1e-6 and repeat >= 1.0:
            v = np.float32(v * np.float32(repeat)) if v <= 0 else np.float32(v / np.float32(repeat))
        out[t] = v
    return out


def recent_window(tokens, last_n: int = 64):
    """Tail of the token history that penalties look at.  src/sampler.rs:92-95,
    window 64 at src/main.rs:539."""
    return list(tokens)[max(0, len(tokens) - last_n):]


def apply_top_k(logits: np.ndarray, k: int) -> np.ndarray:
    """Entries below the k-th largest value become -inf (ties at the threshold stay);
    k == 0 or k >= n disables.  src/sampler.rs:125-137."""
    out = np.array(logits, dtype=np.float32)
    if k == 0 or k >= len(out):
        return out
    thr = np.sort(out)[::-1][k - 1]
    out[out < thr] = -np.inf
    return out


def apply_top_p(logits: np.ndarray, p: float) -> np.ndarray:
    """Softmax over the finite entries, stable sort descending, keep the shortest prefix
    whose cumulative probability exceeds p; the rest become -inf, raw logits are kept.
    p <= 0 or p >= 1 disables.  src/sampler.rs:149-196."""
    out = np.array(logits, dtype=np.float32)
    if p <= 0.0 or p >= 1.0:
        return out
    idx = np.nonzero(out > -np.inf)[0]
    if idx.size == 0:
        return out
    vals = out[idx]
    mx = vals.max()
    total = np.sum(np.exp((vals - mx).astype(np.float64)))
    probs = np.exp(vals - mx).astype(np.float32) / np.float32(total)
    order = np.argsort(-probs, kind="stable")
    cum = np.float32(0.0)
    keep = len(order)
    for n, j in enumerate(order):
        cum = np.float32(cum + probs[j])
        if cum > p:
            keep = n + 1
            break
    out[idx[order[keep:]]] = -np.inf
    return out


def temperature_probs(logits: np.ndarray, temp: float) -> np.ndarray:
    """l/temp, exp(l - max) (0 for -inf), sum in f64, times 1/sum as f32.
    src/sampler.rs:229-249."""
    l = np.array(logits, dtype=np.float32) * np.float32(1.0 / temp)
    mx = l.max()
    e = np.where(l > -np.inf, np.exp(l - mx), 0.0).astype(np.float32)
    inv = np.float32(1.0 / np.sum(e.astype(np.float64)))
    return e * inv


def sample_from_probs(probs: np.ndarray, r: float, acc=np.float32) -> int:
    """Walk indices upward, skipping p <= 0, return the first whose running sum reaches r;
    the last index if none does.  src/sampler.rs:253-266.  The reference keeps the running
    sum in f32 (`acc`); over a vocabulary of 10^5 entries that sum drifts by about 1e-4, so
    tests of large vocabularies pass acc=np.float64, the same walk without the drift."""
    cum = acc(0.0)
    for i, v in enumerate(probs):
        if v <= 0.0:
            continue
        cum = acc(cum + acc(v))
        if r <= cum:
            return i
    return len(probs) - 1


def sample(logits: np.ndarray, temp: float, r: float, top_k: int = 0, top_p: float = 1.0,
           repeat: float = 1.0, frequency: float = 0.0, presence: float = 0.0,
           prev_tokens=()) -> int:
    """penalties -> (greedy if temp < 1e-6) -> top-k -> top-p -> temperature draw with
    the given uniform r in [0,1).  src/sampler.rs:272-290."""
    l = apply_penalties(logits, prev_tokens, repeat, frequency, presence)
    if temp < 1e-6:
        return greedy(l)
    l = apply_top_k(l, top_k)
    l = apply_top_p(l, top_p)
    return sample_from_probs(temperature_probs(l, temp), r)

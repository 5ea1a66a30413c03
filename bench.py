#!/usr/bin/env python3
"""Decode and prefill throughput of the Qwen2.5-7B-shaped model with random weights on one
MI355X: `python bench.py [--gpus 1] [--steps K] [--warmup W]` prints one JSON line.

A step is one decode step of the whole batch (model, sampling, feeding the token back),
replayed from the captured HIP graph; `value` is decoded tokens per second at batch 8 with
unequal prompt lengths up to 2048 in a context of 4096.  The line also carries the prefill
of 2,048 tokens, the decode step's share of the HBM roofline, and further points: decode at
batch 1 and 64, decode at batch 8 with contexts up to 16k and 30k, prefills of 512 and 16,384
tokens.  Fractions are of the published peaks; beside them stands what this GPU gave, just
before, to a plain streaming read and to a register-resident loop of matrix-core products
(`measured_peak`).  `--breakdown` adds the time of every kernel of one decode step.
"""
from __future__ import annotations

import argparse
import gc
import json
import statistics
import sys
import time

HBM_GBS = 8000.0          # MI355X HBM3E, GB/s
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}

QWEN25_7B = dict(
    architectures=["Qwen2ForCausalLM"], model_type="qwen2", hidden_act="silu",
    num_hidden_layers=28, hidden_size=3584, num_attention_heads=28, num_key_value_heads=4,
    intermediate_size=18944, vocab_size=152064, rope_theta=1000000.0, rms_norm_eps=1e-6,
    max_position_embeddings=32768, tie_word_embeddings=False, use_sliding_window=False,
    initializer_range=0.02)
# other shapes of the same architecture (for measurements beyond the default run)
SHAPES = {
    "7b": ("Qwen2.5-7B", QWEN25_7B),
    "0.5b": ("Qwen2.5-0.5B", dict(QWEN25_7B, num_hidden_layers=24, hidden_size=896, num_attention_heads=14,
                                  num_key_value_heads=2, intermediate_size=4864, vocab_size=151936,
                                  tie_word_embeddings=True)),
    "1.5b": ("Qwen2.5-1.5B", dict(QWEN25_7B, num_hidden_layers=28, hidden_size=1536, num_attention_heads=12,
                                  num_key_value_heads=2, intermediate_size=8960, vocab_size=151936,
                                  tie_word_embeddings=True)),
    "3b": ("Qwen2.5-3B", dict(QWEN25_7B, num_hidden_layers=36, hidden_size=2048, num_attention_heads=16,
                              num_key_value_heads=2, intermediate_size=11008, vocab_size=151936,
                              tie_word_embeddings=True)),
    "14b": ("Qwen2.5-14B", dict(QWEN25_7B, num_hidden_layers=48, hidden_size=5120, num_attention_heads=40,
                                num_key_value_heads=8, intermediate_size=13824, rms_norm_eps=1e-5)),
    "32b": ("Qwen2.5-32B", dict(QWEN25_7B, num_hidden_layers=64, hidden_size=5120, num_attention_heads=40,
                                num_key_value_heads=8, intermediate_size=27648, rms_norm_eps=1e-5)),
    "72b": ("Qwen2.5-72B", dict(QWEN25_7B, num_hidden_layers=80, hidden_size=8192, num_attention_heads=64,
                                num_key_value_heads=8, intermediate_size=29568, rms_norm_eps=1e-5)),
}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--prompt-max", type=int, default=2048)
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--shape", default="7b", choices=list(SHAPES), help="layer sizes (default: Qwen2.5-7B)")
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the model has")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--no-points", action="store_true", help="skip the further points (batch 1 and 64, long contexts, other prefills)")
    ap.add_argument("--breakdown", action="store_true", help="time every kernel of one decode step (batch of --batch)")
    ap.add_argument("--max-tokens", type=int, default=None,
                    help="cache size in tokens (default: batch x context, or what fits in free memory if less)")
    ap.add_argument("--no-graph", action="store_true")
    ap.add_argument("--only", choices=["decode", "prefill"], help="run one part (for profiles); prints no JSON line")
    return ap.parse_args()


def matrix_params(cfg):
    """(elements of the matrices one decode step reads per layer, of the head)."""
    h, nh, nk = cfg["hidden_size"], cfg["num_attention_heads"], cfg["num_key_value_heads"]
    hd = cfg.get("head_dim") or h // nh
    per_layer = (nh + 2 * nk) * hd * h + h * nh * hd + 3 * cfg["intermediate_size"] * h
    small = (nh + 2 * nk) * hd + 2 * h
    return per_layer, small, cfg["vocab_size"] * h


def decode_bytes(cfg, elem, total_context):
    per_layer, small, head = matrix_params(cfg)
    nk, hd = cfg["num_key_value_heads"], cfg.get("head_dim") or cfg["hidden_size"] // cfg["num_attention_heads"]
    L = cfg["num_hidden_layers"]
    weights = (L * per_layer + head) * elem + (L * small + cfg["hidden_size"]) * 4
    kv = total_context * 2 * L * nk * hd * elem
    return weights + kv


def prefill_flops(cfg, t):
    per_layer, _, head = matrix_params(cfg)
    nh, hd = cfg["num_attention_heads"], cfg.get("head_dim") or cfg["hidden_size"] // cfg["num_attention_heads"]
    L = cfg["num_hidden_layers"]
    gemm = 2.0 * t * L * per_layer + 2.0 * head          # the head runs on the one wanted row
    attn = L * 2.0 * nh * hd * t * (t + 1)               # causal: QK^T and PV over t(t+1)/2 pairs
    return gemm + attn


def prompt_lengths(batch, prompt_max, seed=0):
    import numpy as np
    rng = np.random.default_rng(seed)
    lens = [int(x) for x in rng.integers(1, prompt_max + 1, size=batch)]
    lens[0] = prompt_max
    return lens


def measure_peaks():
    """(GB/s of a plain streaming read of 4 GB, FLOP/s of a register-resident bfloat16 MFMA loop)
    on this GPU now: the best of three after a warm-up."""
    import torch
    from minfer_amd.kernels import ops
    buf = torch.empty(1 << 30, dtype=torch.int32, device="cuda")      # 4 GB, beyond every cache
    buf.zero_()
    best_bw = best_fl = 0.0
    for i in range(4):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(4):
            ops.probe_read(buf)
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / 4
        if i:
            best_bw = max(best_bw, buf.numel() * 4 / dt / 1e9)
    for i in range(4):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        flops = ops.probe_mfma(20000)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        if i:
            best_fl = max(best_fl, flops / dt)
    del buf
    return best_bw, best_fl


def kernel_breakdown(eng, cfg, batch, prompt_max):
    """Runs one eager decode step of `batch` sequences with an event behind every launch and
    returns [(launch name, calls, microseconds in total)] by total time.  A long matrix-core loop is
    queued first so that the host, which is slower than the GPU at this, stays ahead."""
    import numpy as np
    import torch
    from minfer_amd.kernels import ops
    rng = np.random.default_rng(1)
    lens = prompt_lengths(batch, prompt_max)
    slots = [eng.new_sequence() for _ in lens]
    for s, n in zip(slots, lens):
        eng.step([s], [[int(t) for t in rng.integers(0, cfg["vocab_size"], size=n)]], [[]])
    toks = [[int(t)] for t in rng.integers(0, cfg["vocab_size"], size=batch)]
    eng.step(slots, toks, "last")                       # warm: tables, workspaces
    ctx = eng.build_context(slots, toks, "last")        # (its upload waits for the stream, so it comes first)
    torch.cuda.synchronize()
    ops.probe_mfma(200000)                              # some 50 ms of work ahead of the step
    ops.start_trace()
    eng.model.forward(ctx)
    rows = ops.stop_trace()
    eng.cache.commit(ctx.new_lengths)
    for s in slots:
        eng.end_sequence(s)
    agg = {}
    for name, us in rows:
        n, t = agg.get(name, (0, 0.0))
        agg[name] = (n + 1, t + us)
    return sorted(((k, n, t) for k, (n, t) in agg.items()), key=lambda r: -r[2])


def run_decode(eng, cfg, batch, prompt_max, steps, warmup, use_graph, elem, seed=0):
    """Prefills `batch` unequal prompts (untimed), then times `steps` decode steps."""
    import numpy as np
    import torch
    from minfer_amd.sampling import Sampler, SamplingParams
    rng = np.random.default_rng(1)
    lens = prompt_lengths(batch, prompt_max, seed)
    prompts = [[int(t) for t in rng.integers(0, cfg["vocab_size"], size=n)] for n in lens]
    slots = [eng.new_sequence() for _ in prompts]
    first, group, toks = [], [], 0
    for i, p in enumerate(prompts):            # prompts in steps of at most 8192 tokens
        group.append(i)
        toks += len(p)
        if toks >= 8192 or i == len(prompts) - 1:
            lg = eng.step([slots[j] for j in group], [prompts[j] for j in group], "last")
            first += torch.argmax(lg, dim=-1).cpu().tolist()
            group, toks = [], 0
    sampler = Sampler(SamplingParams.greedy())
    sess = eng.decode_session(batch, prompt_max + warmup + steps + 8, sampler, use_graph=use_graph)
    sess.bind(slots, first, list(range(batch)), [1] * batch)
    def run(n):
        """n decode steps the way the generation loop runs them: the next step is started before
        the tokens of the one before are read."""
        pending = sess.launch()
        for _ in range(n - 1):
            ahead = sess.launch()
            sess.collect(pending)
            pending = ahead
        sess.collect(pending)

    if warmup:
        run(warmup)
    ctx_start = sum(eng.length(s) for s in slots)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    run(steps)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ctx_end = sum(eng.length(s) for s in slots)
    for s in slots:
        eng.end_sequence(s)
    nbytes = decode_bytes(cfg, elem, (ctx_start + ctx_end) / 2.0)
    return dict(tok_s=batch * steps / dt, ms=dt / steps * 1e3, gbs=nbytes / (dt / steps) / 1e9, bytes=nbytes)


def run_prefill(eng, cfg, n_tokens, repeats=5):
    import numpy as np
    import torch
    rng = np.random.default_rng(2)
    prompt = [int(t) for t in rng.integers(0, cfg["vocab_size"], size=n_tokens)]
    times = []
    for i in range(repeats + 2):
        s = eng.new_sequence()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        eng.step([s], [prompt], "last")
        torch.cuda.synchronize()
        if i >= 2:
            times.append(time.perf_counter() - t0)
        eng.end_sequence(s)
    return statistics.median(times)


def main() -> int:
    a = parse()
    if a.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {a.gpus} is not supported (this engine runs on a single MI355X)")
        return 2
    import torch
    from minfer_amd import LLM, Engine
    shape_name, shape = SHAPES[a.shape]
    full_layers = shape["num_hidden_layers"]
    a.layers = a.layers or full_layers
    cfg = dict(shape, num_hidden_layers=a.layers)
    dtype = {"bf16": "bfloat16", "fp32": "float32"}[a.dtype]
    elem = 2 if a.dtype == "bf16" else 4
    points_on = not (a.no_points or a.only)
    batches = [a.batch] + ([1, 64] if points_on else [])
    read_gbs, mfma_flops = measure_peaks()
    # the cache: the batch's contexts, or what the memory left by the weights holds if that is less
    llm = LLM(config=cfg, random_weights=True, weight_seed=0, dtype=dtype, n_ctx=a.context,
              n_slots=max(batches), max_tokens=a.max_tokens)
    eng = llm.engine
    plan = llm.cache_plan
    print(f"cache: {plan['tokens']} tokens ({plan['bytes'] / 2**30:.1f} GiB) for {plan['slots']} slots of "
          f"{plan['context']}" + (" (limited by free memory)" if plan["limited_by_memory"] else ""), file=sys.stderr)
    if a.only == "decode":
        r = run_decode(eng, cfg, a.batch, a.prompt_max, a.steps, a.warmup, not a.no_graph, elem)
        print(f"decode batch {a.batch}: {r['tok_s']:.1f} tok/s, {r['ms']:.3f} ms/step, {r['gbs']:.0f} GB/s")
        return 0
    if a.only == "prefill":
        s = run_prefill(eng, cfg, a.prefill_tokens)
        print(f"prefill {a.prefill_tokens} tokens: {s * 1e3:.2f} ms, {a.prefill_tokens / s:.0f} tok/s")
        return 0
    main_run = run_decode(eng, cfg, a.batch, a.prompt_max, a.steps, a.warmup, not a.no_graph, elem)
    pre_s = run_prefill(eng, cfg, a.prefill_tokens)
    points = {}
    half = (max(16, a.steps // 2), max(4, a.warmup // 2))
    for b in batches[1:]:
        r = run_decode(eng, cfg, b, a.prompt_max, half[0], half[1], not a.no_graph, elem)
        points[f"decode_b{b}"] = round(r["tok_s"], 1)
    breakdown = kernel_breakdown(eng, cfg, a.batch, a.prompt_max) if a.breakdown else None
    if points_on:
        points["prefill_512"] = round(512 / run_prefill(eng, cfg, 512, repeats=3), 1)
        # long contexts: 8 sequences of up to 32,768 tokens, in the same cache where it holds them,
        # else in one of their own on the same weights (the first one is given back before)
        need = 8 * 32768
        long_eng = eng
        if eng.capacity_tokens() < need:
            from minfer_amd.engine.engine import tokens_that_fit
            llm.engine = eng = None
            gc.collect()
            torch.cuda.empty_cache()
            long_eng = Engine(llm.model, max_tokens=min(need, tokens_that_fit(llm.model)), max_seqs=8)
        points["prefill_16384"] = round(16384 / run_prefill(long_eng, cfg, 16384, repeats=2), 1)
        for ctx_max, tag in ((16384, "16k"), (30000, "30k")):
            if long_eng.capacity_tokens() < 8 * (ctx_max + 64 + half[0] + half[1]):
                points[f"decode_b8_ctx{tag}"] = None         # the memory left by the weights does not hold it
                continue
            r = run_decode(long_eng, cfg, 8, ctx_max, half[0], half[1], not a.no_graph, elem, seed=3)
            points[f"decode_b8_ctx{tag}"] = round(r["tok_s"], 1)
    flops = prefill_flops(cfg, a.prefill_tokens)
    out = {
        "metric": f"decode tok/s, {shape_name} shape, batch {a.batch}", "value": round(main_run["tok_s"], 1),
        "unit": "tokens/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(main_run["ms"], 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": a.dtype, "data": "synthetic",
        "config": {"model": f"{shape_name} shape, random weights", "layers": a.layers, "layers_full": full_layers,
                   "hidden": cfg["hidden_size"], "heads": cfg["num_attention_heads"],
                   "kv_heads": cfg["num_key_value_heads"], "head_dim": cfg["hidden_size"] // cfg["num_attention_heads"],
                   "intermediate": cfg["intermediate_size"], "vocab": cfg["vocab_size"],
                   "global_batch": a.batch, "seq_len": a.context, "prompt_max": a.prompt_max,
                   "prefill_tokens": a.prefill_tokens, "parallelism": "single GPU",
                   "decode_graph": not a.no_graph, "cache_tokens": plan["tokens"],
                   "tiled_weight_copies_gib": round(getattr(llm.model, "decode_copy_bytes", 0) / 2 ** 30, 2)},
        "prefill": {"value": round(a.prefill_tokens / pre_s, 1), "tokens": a.prefill_tokens,
                    "ms": round(pre_s * 1e3, 3), "frac": round(flops / pre_s / PEAK_FLOPS[a.dtype], 4),
                    "measured_peak": round(mfma_flops / 1e12, 1), "unit": "TFLOP/s (bf16 MFMA loop in registers)"},
        "roofline": {"bound": "hbm", "achieved": round(main_run["gbs"], 1), "peak": HBM_GBS, "unit": "GB/s",
                     "frac": round(main_run["gbs"] / HBM_GBS, 4), "measured_peak": round(read_gbs, 1),
                     "frac_of_measured": round(main_run["gbs"] / read_gbs, 4)},
        "points": points,
    }
    if breakdown is not None:
        total = sum(t for _, _, t in breakdown)
        print(f"one decode step of batch {a.batch}, kernel by kernel ({total:.0f} us):", file=sys.stderr)
        for name, n, t in breakdown:
            print(f"  {name:46s} {n:4d} x {t / n:8.1f} us = {t:9.1f} us  {100 * t / total:5.1f} %", file=sys.stderr)
        out["breakdown_us"] = {name: round(t, 1) for name, n, t in breakdown}
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())

"""Generation on the GPU through the entry points: greedy and sampled tokens against the
plain implementation, the captured decode step against the eager one, long decoding, the
first tokens of a sequence, the command line, and trace replay as a program."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

import plain_qwen2 as pq
from minfer_amd.sampling import uniform
from replays import (batch_steps, compare, plain_logits, requests_for, run_steps, tail_steps, whole_steps)
from tiny import TINIES, random_tokens, write_tiny

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("gen")
    return {n: write_tiny(tmp, n, seed=7) for n in TINIES}


def plain_generate(plain, prompt, n, temp, seed, key, **opts):
    seq, out = list(prompt), []
    for s in range(n):
        logits = plain.forward(seq)[-1].astype(np.float32)
        t = pq.sample(logits, temp, uniform(seed, key, s), opts.get("top_k", 40), opts.get("top_p", 0.95),
                      opts.get("repeat", 1.1), 0.0, 0.0, pq.recent_window(seq))
        out.append(t)
        seq.append(t)
    return out


@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_and_sampled_generation_match_plain(folders, name):
    from minfer_amd import LLM
    plain = pq.PlainQwen2.from_folder(folders[name])
    vocab = TINIES[name]["vocab_size"]
    lens = (5, 9, 13) if name == "A" else (1, 7, 31, 64)
    steps = 8 if name == "A" else 16
    prompts = [random_tokens(vocab, n, 10 + i) for i, n in enumerate(lens)]
    llm = LLM(folders[name], dtype="float32", n_ctx=128, n_slots=4)
    for temp in (0.0, 0.8):
        eager = llm.generate(prompts, max_new=steps, temp=temp, seed=1, stop_tokens=[], use_graph=False)
        graph = llm.generate(prompts, max_new=steps, temp=temp, seed=1, stop_tokens=[], use_graph=True)
        assert eager.tokens == graph.tokens
        for i, p in enumerate(prompts):
            assert graph.tokens[i] == plain_generate(plain, p, steps, temp, 1, i), (name, temp, i)
    # bfloat16: the same tokens from the captured and the eager step
    lb = LLM(folders[name], dtype="bfloat16", n_ctx=128, n_slots=4)
    a = lb.generate(prompts, max_new=steps, temp=0.0, repeat_penalty=1.0, stop_tokens=[], use_graph=False)
    b = lb.generate(prompts, max_new=steps, temp=0.0, repeat_penalty=1.0, stop_tokens=[], use_graph=True)
    assert a.tokens == b.tokens and all(len(t) == steps for t in b.tokens)
    assert not lb.engine.cache.live_slots()


def test_captured_step_with_room_for_long_sequences_shares_the_key_splits(tmp_path):
    """A session made for 8,320 positions: the captured decode step's attention deals its key splits
    out by the sequences' lengths (eight sequences of 1 to 300 tokens here; most splits of a share
    lie past the keys), the eager step, which knows the lengths, gives every sequence the same
    number.  The same tokens from both, and the logits of the plain implementation."""
    from minfer_amd import LLM, config_from_dict, write_random_model
    from minfer_amd.kernels import ops
    cfg = dict(TINIES["A"], max_position_embeddings=8320)
    folder = str(tmp_path / "tiny_A_long")
    write_random_model(folder, config_from_dict(cfg), 11)
    places, splits = ops.decode_split_plan(8, cfg["num_key_value_heads"], 2, 8320)
    assert places > splits > 1, "this session is meant to share the splits out"
    lens = (5, 300, 33, 64, 129, 70, 1, 200)
    prompts = [random_tokens(cfg["vocab_size"], n, 30 + i) for i, n in enumerate(lens)]
    llm = LLM(folder, dtype="bfloat16", n_ctx=8320, n_slots=8)
    eager = llm.generate(prompts, max_new=6, temp=0.0, repeat_penalty=1.0, stop_tokens=[], use_graph=False)
    graph = llm.generate(prompts, max_new=6, temp=0.0, repeat_penalty=1.0, stop_tokens=[], use_graph=True)
    assert eager.tokens == graph.tokens and all(len(t) == 6 for t in graph.tokens)
    # the decode step itself, through the session, against the plain implementation
    plain = pq.PlainQwen2.from_folder(folder)
    eng = llm.engine
    from minfer_amd.sampling import Sampler, SamplingParams
    slots = [eng.new_sequence() for _ in prompts]
    eng.step(slots, prompts, [[] for _ in prompts])
    sess = eng.decode_session(len(prompts), 8320, Sampler(SamplingParams(temp=0.0, repeat_penalty=1.0)), use_graph=True)
    sess.bind(slots, [t[0] for t in graph.tokens], list(range(len(prompts))), [1] * len(prompts))
    sess.set_windows(prompts)
    for step in range(1, 4):                   # eager, captured, replayed
        sampled = sess.step()
        assert sampled == [t[step] for t in graph.tokens]
        got = sess.last_logits.float().cpu().numpy()
        for i, p in enumerate(prompts):
            want = plain.forward(list(p) + graph.tokens[i][:step])[-1]
            sd = want.std()
            err = got[i] - want
            assert np.sqrt((err ** 2).mean()) <= 0.01 * sd and np.abs(err).max() <= 0.055 * sd, (step, i)
    for s in slots:
        eng.end_sequence(s)
    assert not eng.cache.live_slots()


def test_stop_tokens_end_sequences_early_and_batches_follow_each_other(folders):
    from minfer_amd import LLM
    plain = pq.PlainQwen2.from_folder(folders["A"])
    prompts = [random_tokens(512, n, 30 + i) for i, n in enumerate((4, 11, 6, 20, 3))]
    llm = LLM(folders["A"], dtype="float32", n_ctx=64, n_slots=2)
    free = llm.generate(prompts, max_new=12, temp=0.8, seed=5, stop_tokens=[])
    assert free.batches == [[0, 1], [2, 3], [4]]
    # declare each request's 4th token (if new to it) a stop token for everyone
    stops = {t[3] for t in free.tokens}
    res = llm.generate(prompts, max_new=12, temp=0.8, seed=5, stop_tokens=sorted(stops))
    for i, p in enumerate(prompts):
        want = plain_generate(plain, p, 12, 0.8, 5, i)
        cut = next((j for j, t in enumerate(want) if t in stops), 12)
        assert res.tokens[i] == want[:cut]
        assert res.finish_reasons[i] == ("stop" if cut < 12 else "length")
    llm.engine.cache.check_invariants()


def test_long_decoding_crosses_pages(folders):
    """300 decode steps after a short prompt, through the captured step, teacher-forced
    against the plain implementation at a few places."""
    from minfer_amd import LLM
    plain = pq.PlainQwen2.from_folder(folders["B"])
    llm = LLM(folders["B"], dtype="float32", n_ctx=512, n_slots=2)
    prompts = [random_tokens(1000, 3, 40), random_tokens(1000, 62, 41)]
    res = llm.generate(prompts, max_new=300, temp=0.9, seed=2, stop_tokens=[])
    assert [len(t) for t in res.tokens] == [300, 300]
    for i, p in enumerate(prompts):
        seq = list(p) + res.tokens[i]
        full = plain.forward(seq[:-1]).astype(np.float32)
        for s in (0, 1, 2, 61, 62, 63, 64, 65, 127, 128, 199, 256, 299):
            window = pq.recent_window(seq[:len(p) + s])
            t = pq.sample(full[len(p) + s - 1], 0.9, uniform(2, i, s), 40, 0.95, 1.1, 0, 0, window)
            assert t == res.tokens[i][s], (i, s)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens_of_a_sequence(folders, dtype):
    """Prompts of one token, the first decoded token, a prompt that ends on a page edge."""
    from minfer_amd import Engine, load_model
    plain = pq.PlainQwen2.from_folder(folders["C"])
    eng = Engine(load_model(folders["C"], dtype=dtype), max_tokens=64 * 6, poison_cache=True)
    reqs = requests_for(777, (1, 2, 64, 65), seed=9)
    ref = plain_logits(plain, reqs)
    steps = []
    ids = list(reqs)
    steps.append(dict(step=0, entries=[dict(id=r, tokens=reqs[r][:1] if len(reqs[r]) < 3 else reqs[r][:-1],
                                            want=[0] if len(reqs[r]) < 3 else [len(reqs[r]) - 2])
                                       for r in ids], end=["r0"]))
    steps.append(dict(step=1, entries=[dict(id=r, tokens=reqs[r][-1:], want=[0]) for r in ids[1:]], end=ids[1:]))
    compare(run_steps(eng, steps), ref, dtype, "first tokens")


def test_captured_steps_survive_growth_of_shared_scratch(folders):
    """A captured decode step holds the addresses of the shared scratch buffers and of the
    rotation table.  When a later, larger job makes them grow, the earlier graphs must go on
    working: what was outgrown stays allocated."""
    import torch
    from minfer_amd import LLM
    from minfer_amd.kernels import ops
    vocab = TINIES["C"]["vocab_size"]
    llm = LLM(folders["C"], dtype="bfloat16", n_ctx=1024, n_slots=4)
    prompts = [random_tokens(vocab, n, 40 + i) for i, n in enumerate((30, 70))]
    first = llm.generate(prompts, max_new=12, temp=0.0, stop_tokens=[]).tokens       # captures graphs for 2 sequences
    held = {k: v for k, v in ops._workspaces.items()}
    for (tag, dev), w in held.items():                    # somebody needs more of every scratch buffer
        ops.workspace(tag, w.numel() * 2 + 1, w.device)
    junk = [torch.full((w.numel(),), float("nan"), device=w.device) for w in held.values()]   # would land in freed blocks
    long_prompt = [random_tokens(vocab, 700, 50)]
    llm.generate(long_prompt, max_new=4, temp=0.0, stop_tokens=[])        # a longer sequence: the rotation table grows
    again = llm.generate(prompts, max_new=12, temp=0.0, stop_tokens=[]).tokens       # the old graphs replay
    eager = llm.generate(prompts, max_new=12, temp=0.0, stop_tokens=[], use_graph=False).tokens
    assert again == first == eager
    del junk


def test_command_line(folders, tmp_path):
    env = dict(os.environ, PYTHONPATH=ROOT)
    exe = [sys.executable, os.path.join(ROOT, "bin", "minfer")]
    r = subprocess.run(exe + [folders["A"], "--prompt-tokens", "5,6,7;9,10", "--greedy", "--repeat-penalty", "1.0",
                              "-n", "5", "--dtype", "float32", "--n-ctx", "64", "--stop-token", "100000"],
                       capture_output=True, text=True, env=env, timeout=300)
    assert r.returncode == 0, r.stderr
    lines = [l for l in r.stdout.strip().splitlines() if l]
    plain = pq.PlainQwen2.from_folder(folders["A"])
    for line, prompt in zip(lines, ([5, 6, 7], [9, 10])):
        seq = list(prompt)
        for t in (int(x) for x in line.split(",")):
            assert t == pq.greedy(plain.forward(seq)[-1])
            seq.append(t)
    assert "Prefill: 5 tokens" in r.stderr and "Generated:" in r.stderr and "Total:" in r.stderr
    cfg = tmp_path / "c.json"
    cfg.write_text(json.dumps(TINIES["B"]))
    r = subprocess.run(exe + ["--config", str(cfg), "--random-weights", "--prompt-tokens", "1,2,3", "--max-new", "4",
                              "--temp", "0.8", "--seed", "3"], capture_output=True, text=True, env=env, timeout=300)
    assert r.returncode == 0, r.stderr
    # the same options through the Python entry point: the same random weights, the same draws
    from minfer_amd import LLM
    same = LLM.random(TINIES["B"], seed=0, dtype="bfloat16", n_ctx=4096, n_slots=1).generate(
        [[1, 2, 3]], max_new=4, temp=0.8, seed=3)
    assert [int(x) for x in r.stdout.strip().split(",") if x] == same.tokens[0] and 1 <= len(same.tokens[0]) <= 4
    # ... and they are the weights of the folder that the same configuration and seed write
    folder_b = write_tiny(tmp_path, "B", seed=0)
    from_folder = LLM(folder_b, dtype="bfloat16", n_ctx=4096, n_slots=1).generate([[1, 2, 3]], max_new=4, temp=0.8, seed=3)
    assert from_folder.tokens == same.tokens
    r = subprocess.run(exe + [folders["A"], "--bogus"], capture_output=True, text=True, env=env, timeout=60)
    assert r.returncode == 1 and "unknown option --bogus" in r.stderr and "USAGE" in r.stderr
    r = subprocess.run(exe + [folders["A"], "--prompt-tokens", "1", "--temp"], capture_output=True, text=True,
                       env=env, timeout=60)
    assert r.returncode == 1 and "requires a value" in r.stderr


def test_debug_switches_change_no_token(folders):
    """MF_DEBUG_SYNC=1 (a synchronisation and an error check behind every launch, its name
    printed) and MF_TIMING=1 (a token's time split into forward and sampling): the same tokens as
    without them, and the lines they promise (the reference's MINFER_CUDA_DEBUG and
    MINFER_TIMING, src/cuda.rs:378-395 and src/main.rs:552-609 of yusiwen/minfer)."""
    exe = [sys.executable, os.path.join(ROOT, "bin", "minfer"), folders["A"], "--prompt-tokens", "5,6,7;9,10,11,12",
           "--temp", "0.7", "--seed", "5", "-n", "6", "--n-ctx", "64", "--stop-token", "100000"]
    runs = {}
    for switch in ("", "MF_DEBUG_SYNC", "MF_TIMING"):
        env = dict(os.environ, PYTHONPATH=ROOT)
        env.pop("MF_DEBUG_SYNC", None)
        env.pop("MF_TIMING", None)
        if switch:
            env[switch] = "1"
        r = subprocess.run(exe, capture_output=True, text=True, env=env, timeout=300)
        assert r.returncode == 0, r.stderr
        runs[switch] = r
    plain_out = runs[""].stdout
    assert len(plain_out.strip().splitlines()) == 2
    assert runs["MF_DEBUG_SYNC"].stdout == plain_out and runs["MF_TIMING"].stdout == plain_out
    ok = [l for l in runs["MF_DEBUG_SYNC"].stderr.splitlines() if l.startswith("[minfer_amd] ") and l.endswith(" OK")]
    assert len(ok) > 50 and any("attn" in l for l in ok) and any("gemm" in l for l in ok) and any("sample" in l or "argmax" in l for l in ok)
    assert " OK" not in runs[""].stderr and "[MF_TIMING]" not in runs[""].stderr
    timing = [l for l in runs["MF_TIMING"].stderr.splitlines() if l.startswith("[MF_TIMING]")]
    assert len(timing) == 1 and "sample" in timing[0] and "forward" in timing[0] and "ms/tok" in timing[0]


def test_trace_names_every_launch_of_a_step(folders):
    """`ops.start_trace` / `stop_trace`: one (name, microseconds) entry per kernel launch, in launch
    order.  A 32-bit prompt step of the two-layer model is: the embedding; per layer norm, q|k|v,
    rotation + cache write, attention, o, norm, gate|up, SwiGLU, down, with the wanted rows
    gathered before the last feed-forward; final norm; head."""
    from minfer_amd import Engine, load_model
    from minfer_amd.kernels import ops
    eng = Engine(load_model(folders["A"], dtype="float32"), max_tokens=128)
    s = eng.new_sequence()
    eng.step([s], [[1, 2, 3]], "last")                  # builds tables and workspaces outside the trace
    eng.end_sequence(s)
    s = eng.new_sequence()
    ops.start_trace()
    eng.step([s], [[4, 5, 6, 7, 8]], "last")
    entries = ops.stop_trace()
    eng.end_sequence(s)
    layer = ["rmsnorm", "gemm_f32", "rope_kvwrite", "attn_tokens_f32", "gemm_f32", "rmsnorm", "gemm_f32", "swiglu", "gemm_f32"]
    last = layer[:5] + ["gather_rows"] + layer[5:]
    want = ["embed"] + layer + last + ["rmsnorm", "gemm_f32"]
    assert [name.split()[0] for name, _ in entries] == want
    assert all(us >= 0.0 for _, us in entries) and sum(us for _, us in entries) > 0.0
    assert ops.stop_trace() == []                       # nothing is recorded once stopped
    s = eng.new_sequence()
    eng.step([s], [[1]], "last")
    eng.end_sequence(s)
    assert ops.stop_trace() == []


def test_cache_is_sized_from_the_free_memory_when_that_is_less(folders, monkeypatch):
    """With little device memory free, the cache takes what fits instead of slots x context
    (`cache_plan` says so), generation plans its batches by that capacity, and with no room at all
    the error says why."""
    import torch
    from minfer_amd import LLM
    from minfer_amd.cache import CacheError
    from minfer_amd.engine.engine import RESERVE_BYTES_MIN
    real = torch.cuda.mem_get_info
    total = real()[1]
    reserve = max(RESERVE_BYTES_MIN, int(0.06 * total)) + 8192 * 64 * 4 * 12
    per_token = 2 * 2 * 2 * 16 * 2                      # two layers, K and V, two kv heads of 16, bfloat16
    state = {"free": reserve + 5 * 64 * per_token + 100}
    monkeypatch.setattr(torch.cuda, "mem_get_info", lambda device=None: (state["free"], total))
    llm = LLM(folders["A"], dtype="bfloat16", n_ctx=128, n_slots=4)
    plan = llm.cache_plan
    assert plan["limited_by_memory"] and plan["fits"] == 5 * 64 and plan["tokens"] == 5 * 64
    assert plan["bytes_per_token"] == per_token and llm.engine.capacity_tokens() == 320
    prompts = [random_tokens(512, n, 60 + i) for i, n in enumerate((70, 30, 90, 20))]      # 2 + 1 + 2 + 1 pages and growth
    res = llm.generate(prompts, max_new=40, temp=0.0, stop_tokens=[])
    assert [len(t) for t in res.tokens] == [min(40, 128 - len(p) + 1) for p in prompts]    # 128 positions end the longest
    assert len(res.batches) > 1, "four requests cannot be live together in five pages"
    monkeypatch.setattr(torch.cuda, "mem_get_info", real)
    roomy = LLM(folders["A"], dtype="bfloat16", n_ctx=128, n_slots=4)
    assert not roomy.cache_plan["limited_by_memory"] and roomy.cache_plan["tokens"] == 4 * 128
    assert roomy.generate(prompts, max_new=40, temp=0.0, stop_tokens=[]).tokens == res.tokens
    state["free"] = reserve + 10
    monkeypatch.setattr(torch.cuda, "mem_get_info", lambda device=None: (state["free"], total))
    with pytest.raises(CacheError, match="no room for a cache"):
        LLM(folders["A"], dtype="bfloat16", n_ctx=128, n_slots=4)


def replay_program(folder, dtype, steps, out_dir, max_tokens):
    """Runs bin/trace_run as a program; sends each step only after the last `done`."""
    exe = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
           "--out", out_dir, "--max-tokens", str(max_tokens)]
    p = subprocess.Popen(exe, stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True, bufsize=1)
    pos, rows = {}, {}
    vocab = json.load(open(os.path.join(folder, "config.json")))["vocab_size"]
    try:
        for st in steps:
            p.stdin.write(json.dumps(st) + "\n")
            p.stdin.flush()
            assert p.stdout.readline().strip() == f"done {st['step']}"
            n_want = sum(len(e["want"]) for e in st["entries"])
            path = os.path.join(out_dir, f"{st['step']}.f32")
            if n_want:
                arr = np.fromfile(path, dtype="<f4").reshape(n_want, vocab)
                r = 0
                for e in st["entries"]:
                    for w in e["want"]:
                        rows[(e["id"], pos.get(e["id"], 0) + w)] = arr[r]
                        r += 1
            else:
                assert not os.path.exists(path)
            for e in st["entries"]:
                pos[e["id"]] = pos.get(e["id"], 0) + len(e["tokens"])
        p.stdin.close()
        assert p.wait(timeout=60) == 0
    finally:
        if p.poll() is None:
            p.kill()
    return rows


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(folders, tmp_path, dtype):
    plain = pq.PlainQwen2.from_folder(folders["B"])
    reqs = requests_for(1000, (1, 7, 31, 64, 90), seed=8)
    ref = plain_logits(plain, reqs)
    ids = list(reqs)
    # peak: the batch of three at its end, each request rounded up to 64
    peak = max(sum((len(reqs[r]) + 63) // 64 * 64 for r in b) for b in (ids[:3], ids[3:]))
    plans = {"whole": whole_steps(reqs), "tail": tail_steps(reqs), "batches": batch_steps(reqs, [ids[:3], ids[3:]])}
    # a step that wants nothing writes no file
    plans["batches"][0]["entries"][0]["want"] = []
    for what, steps in plans.items():
        out = tmp_path / f"{dtype}_{what}"
        rows = replay_program(folders["B"], dtype, steps, str(out), peak if what == "batches" else 128)
        compare(rows, ref, dtype, f"trace_run {what}")

"""Shared helpers of the replay tests: requests, the ways of cutting them into steps (whole,
the last tokens one by one, unequal batches, prompts in portions), and the comparison with the
plain implementation."""
from __future__ import annotations

import numpy as np

from tiny import random_tokens

# bfloat16 logits, as fractions of the logits' standard deviation over the vocabulary.
# bfloat16 keeps 8 bits (relative rounding error 2^-9/sqrt(3) = 0.11 % rms) and a run rounds
# activations about eight times per layer, so the error of a logit is a sum of many small
# independent terms: its rms over the vocabulary is what the size of the model fixes (measured
# 0.3..0.8 % from 64 to 3584 wide), while its maximum grows with the number of entries looked
# at (4.9 sigma at 152064).  Both are bounded: rms 1 %, maximum 5.5 %.
BF16_RMS = 0.01
BF16_MAX = 0.055
F32_ABS = 1e-4
# The tiny configurations (up to three layers) are all held to these figures.  At the 7B widths a
# single layer already comes close to them, and every further layer adds roundings of its own,
# independent of the others': the error's rms grows about with the root of the depth.  Measured at
# those widths, worst row of five requests: the engine's own composition run on host stand-ins that
# round at the same places and compute in 64 bits in between, so that nothing but the roundings
# separates it from the plain implementation, differs from it by 0.81 % rms at one layer and
# 1.40 % at four; the GPU engine by 0.83 % and 1.48 %.  A test of a deeper model at such widths
# passes its depth and is held to the figures above times sqrt(layers).


def bf16_depth_factor(layers: int) -> float:
    return max(1.0, float(layers) ** 0.5)


def requests_for(vocab: int, lengths, seed: int = 0):
    return {f"r{i}": random_tokens(vocab, n, seed * 100 + i) for i, n in enumerate(lengths)}


def plain_logits(plain, requests):
    return {rid: plain.forward(toks) for rid, toks in requests.items()}


def whole_steps(requests):
    """Each request alone and whole: one step with all its tokens, all logits wanted."""
    steps = []
    for rid, toks in requests.items():
        steps.append(dict(step=len(steps), entries=[dict(id=rid, tokens=toks, want=list(range(len(toks))))],
                          end=[rid]))
    return steps


def tail_steps(requests, tail: int = 32):
    """First len - tail tokens in one step, then the last `tail` one by one."""
    steps = []
    for rid, toks in requests.items():
        head = max(0, len(toks) - tail)
        if head:
            steps.append(dict(step=len(steps), entries=[dict(id=rid, tokens=toks[:head], want=list(range(head)))],
                              end=[]))
        for i in range(head, len(toks)):
            steps.append(dict(step=len(steps), entries=[dict(id=rid, tokens=[toks[i]], want=[0])],
                              end=[rid] if i == len(toks) - 1 else []))
    return steps


def batch_steps(requests, batches, prompt_frac: float = 0.6):
    """Batches of unequal lengths that start together: prompts (a fraction of each
    request) in one step, then one token each per step; a request whose tokens run out ends
    while the others go on; the next batch starts afterwards, so slots are used again."""
    steps = []
    for batch in batches:
        plen = {rid: max(1, int(len(requests[rid]) * prompt_frac)) for rid in batch}
        done = {rid: plen[rid] for rid in batch}
        ends = [rid for rid in batch if done[rid] == len(requests[rid])]
        steps.append(dict(step=len(steps),
                          entries=[dict(id=rid, tokens=requests[rid][:plen[rid]], want=list(range(plen[rid])))
                                   for rid in batch], end=ends))
        live = [rid for rid in batch if rid not in ends]
        while live:
            entries, ends = [], []
            for rid in live:
                entries.append(dict(id=rid, tokens=[requests[rid][done[rid]]], want=[0]))
                done[rid] += 1
                if done[rid] == len(requests[rid]):
                    ends.append(rid)
            steps.append(dict(step=len(steps), entries=entries, end=ends))
            live = [rid for rid in live if rid not in ends]
    return steps


def chunk_steps(requests, batches, sizes=(2, 50, 64, 1, 17)):
    """Prompts fed in portions.  The requests of a batch go on together; at every step each one
    still alive brings its next portion, whose sizes run through `sizes` with a different start
    for each request, so portions begin and end on and off page edges, a portion of several
    tokens meets a non-empty cache, and one request's single token shares a step with another's
    fifty.  Every position's logits are asked for; a request ends when its tokens run out."""
    steps = []
    for batch in batches:
        done = {rid: 0 for rid in batch}
        turn = {rid: i for i, rid in enumerate(batch)}
        live = list(batch)
        while live:
            entries, ends = [], []
            for rid in live:
                n = min(sizes[turn[rid] % len(sizes)], len(requests[rid]) - done[rid])
                turn[rid] += 1
                entries.append(dict(id=rid, tokens=requests[rid][done[rid]:done[rid] + n], want=list(range(n))))
                done[rid] += n
                if done[rid] == len(requests[rid]):
                    ends.append(rid)
            steps.append(dict(step=len(steps), entries=entries, end=ends))
            live = [rid for rid in live if rid not in ends]
    return steps


def run_steps(engine, steps):
    """Drives Engine.step with trace steps; returns {(request, position): logits row}."""
    slots, pos, rows = {}, {}, {}
    for st in steps:
        ents = st["entries"]
        for e in ents:
            if e["id"] not in slots:
                slots[e["id"]] = engine.new_sequence()
                pos[e["id"]] = 0
        logits = engine.step([slots[e["id"]] for e in ents], [e["tokens"] for e in ents],
                             [e["want"] for e in ents]).cpu().numpy()
        r = 0
        for e in ents:
            for w in e["want"]:
                rows[(e["id"], pos[e["id"]] + w)] = logits[r]
                r += 1
            pos[e["id"]] += len(e["tokens"])
        assert r == logits.shape[0]
        for rid in st["end"]:
            engine.end_sequence(slots.pop(rid))
        engine.cache.check_invariants()
    return rows


def compare(rows, ref, dtype: str, what: str, layers: int = 1):
    """Every produced row against the plain implementation's; names the first bad place.
    `layers`: the model's depth (it scales the bfloat16 bound beyond three layers)."""
    assert rows, "nothing was produced"
    worst = 0.0
    depth = bf16_depth_factor(layers)
    for (rid, p), got in sorted(rows.items()):
        want = ref[rid][p]
        diff = got.astype(np.float64) - want
        err = float(np.abs(diff).max())
        tol = F32_ABS if dtype == "float32" else BF16_MAX * depth * float(want.std())
        assert np.isfinite(got).all(), f"{what}: non-finite logits at request {rid} position {p}"
        assert err <= tol, (f"{what} [{dtype}]: request {rid} position {p} (of {len(ref[rid])}): "
                            f"max abs err {err:.3e} > {tol:.3e}")
        if dtype != "float32":
            rms = float(np.sqrt(np.mean(diff * diff)))
            assert rms <= BF16_RMS * depth * float(want.std()), (
                f"{what} [{dtype}]: request {rid} position {p}: rms err {rms:.3e} > "
                f"{BF16_RMS * depth * float(want.std()):.3e}")
        worst = max(worst, err)
    return worst

"""The generation loop: batches of unequal prompts, stop tokens, sequences that end
earlier, and as many batches one after another as there are requests.

Shape of the reference's loop (src/main.rs:495-598 of yusiwen/minfer): the prompt in one
call, then `sample -> stop? -> append -> forward(one token)`.  A stop token ends the
sequence before it is appended and is not fed back (src/main.rs:568); the bound is the
number of new tokens (src/main.rs:559); a full context ends the sequence with reason
'length' (src/server/chat.rs:117-121).  Prefill and decode are timed apart and the decode
rate excludes the prefill (src/main.rs:505-508,615-623).  Unlike the reference, no forward
is run for a token that will not be followed by another.
"""
from __future__ import annotations

import time
from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional, Sequence

import torch

from ..cache.paged import PAGE
from ..kernels import tuning
from ..sampling.params import REPEAT_LAST_N, SamplingParams
from ..sampling.sampler import Sampler


@dataclass
class GenerationResult:
    tokens: List[List[int]]                 # generated ids per request, stop token not included
    finish_reasons: List[str]               # 'stop' | 'length'
    prefill_tokens: int = 0
    prefill_seconds: float = 0.0
    decode_tokens: int = 0                  # tokens produced by decode steps
    decode_seconds: float = 0.0
    batches: List[List[int]] = field(default_factory=list)   # request indices of each batch
    forward_seconds: float = 0.0            # with MF_TIMING: decode time spent in the model's step
    sample_seconds: float = 0.0             # with MF_TIMING: decode time spent sampling

    @property
    def prefill_rate(self) -> float:
        return self.prefill_tokens / self.prefill_seconds if self.prefill_seconds > 0 else 0.0

    @property
    def decode_rate(self) -> float:
        return self.decode_tokens / self.decode_seconds if self.decode_seconds > 0 else 0.0


def _sync(engine) -> None:
    if getattr(engine, "device", None) is not None and engine.device.type == "cuda":
        torch.cuda.synchronize(engine.device)


def plan_batches(prompt_lengths: Sequence[int], max_new: int, capacity_tokens: int, max_batch: int,
                 max_positions: int) -> List[List[int]]:
    """Requests in order, as many per batch as the cache can hold to their last token (each
    rounded up to whole pages) and as there are slots."""
    batches, cur, used = [], [], 0
    for i, n in enumerate(prompt_lengths):
        if n < 1:
            raise ValueError(f"request {i}: empty prompt")
        if n > max_positions:
            raise ValueError(f"request {i}: prompt of {n} tokens exceeds the model's {max_positions} positions")
        need = (min(n + max_new, max_positions) + PAGE - 1) // PAGE * PAGE
        if need > capacity_tokens:
            raise ValueError(f"request {i}: needs {need} cache tokens, the cache holds {capacity_tokens}")
        if cur and (used + need > capacity_tokens or len(cur) >= max_batch):
            batches.append(cur)
            cur, used = [], 0
        cur.append(i)
        used += need
    if cur:
        batches.append(cur)
    return batches


def generate(engine, prompts: Sequence[Sequence[int]], params: Optional[SamplingParams] = None,
             max_new: int = 512, stop_tokens: Optional[Sequence[int]] = None, max_batch: Optional[int] = None,
             use_graph: bool = True, on_token: Optional[Callable[[int, int], None]] = None,
             n_ctx: Optional[int] = None) -> GenerationResult:
    """Generates up to `max_new` tokens for every prompt (lists of token ids).  `stop_tokens`
    defaults to the model's own; `on_token(request, token)` is called for each emitted token;
    `n_ctx` bounds the positions of one sequence (default: the model's own bound)."""
    params = params or SamplingParams()
    sampler = Sampler(params)
    if stop_tokens is None:
        stop_tokens = engine.stop_tokens()
    stops = set(int(t) for t in stop_tokens)
    n_req = len(prompts)
    result = GenerationResult(tokens=[[] for _ in range(n_req)], finish_reasons=["length"] * n_req)
    if n_req == 0 or max_new <= 0:
        return result
    capacity = engine.capacity_tokens()
    max_batch = min(max_batch or engine.max_seqs, engine.max_seqs)
    limit = min(engine.max_positions, n_ctx) if n_ctx else engine.max_positions
    result.batches = plan_batches([len(p) for p in prompts], max_new, capacity, max_batch, limit)
    dev = engine.device

    held = set()                             # slots this call has taken and not yet given back
    timing = tuning.TIMING
    if timing:
        use_graph = False                    # the split needs a stop between the step and the sampling

    def release(slot: int) -> None:
        held.discard(slot)
        engine.end_sequence(slot)

    def decide(req: int, tok: int, slot: int, live: Dict[int, int], length: Optional[int] = None) -> None:
        """After sampling `tok` for request `req`: stop, emit, or emit and end.  `length` is what
        the sequence held after the step that gave `tok` (default: what it holds now)."""
        if length is None:
            length = engine.length(slot)
        if tok in stops:
            result.finish_reasons[req] = "stop"
        else:
            result.tokens[req].append(tok)
            if on_token:
                on_token(req, tok)
            if len(result.tokens[req]) < max_new and length + 1 <= limit:
                live[req] = slot
                return
            result.finish_reasons[req] = "length"
        release(slot)

    def run_batch(batch: List[int]) -> None:
        slots = {}
        for r in batch:
            slots[r] = engine.new_sequence()
            held.add(slots[r])
        windows = {r: list(prompts[r])[-REPEAT_LAST_N:] for r in batch}
        _sync(engine)
        t0 = time.perf_counter()
        logits = engine.step([slots[r] for r in batch], [list(prompts[r]) for r in batch], "last")
        first = _sample(sampler, logits, batch, [0] * len(batch), [windows[r] for r in batch], dev)
        _sync(engine)
        result.prefill_seconds += time.perf_counter() - t0
        result.prefill_tokens += sum(len(prompts[r]) for r in batch)
        live: Dict[int, int] = {}
        for r, tok in zip(batch, first):
            windows[r] = (windows[r] + [tok])[-REPEAT_LAST_N:]
            decide(r, tok, slots[r], live)
        next_tok = {r: result.tokens[r][-1] for r in live}

        t0 = time.perf_counter()
        while live:
            order = sorted(live)
            if use_graph and hasattr(engine, "decode_session"):
                live = _decode_bound(engine, sampler, params, order, live, next_tok, windows, prompts, result,
                                     max_new, limit, decide)
            else:
                t1 = time.perf_counter()
                logits = engine.step([live[r] for r in order], [[next_tok[r]] for r in order], "last")
                if timing:
                    _sync(engine)
                    t2 = time.perf_counter()
                    result.forward_seconds += t2 - t1
                toks = _sample(sampler, logits, order, [len(result.tokens[r]) for r in order],
                               [windows[r] for r in order], dev)
                if timing:
                    result.sample_seconds += time.perf_counter() - t2
                result.decode_tokens += len(order)
                was, live = live, {}
                for r, tok in zip(order, toks):
                    windows[r] = (windows[r] + [tok])[-REPEAT_LAST_N:]
                    decide(r, tok, was[r], live)
            next_tok = {r: result.tokens[r][-1] for r in live}
        _sync(engine)
        result.decode_seconds += time.perf_counter() - t0

    try:
        for batch in result.batches:
            run_batch(batch)
    finally:
        # whatever ended the loop (an error in a step, in `on_token`, an interrupt): no slot of
        # this call stays taken, so the engine is as free for the next call as before this one
        for slot in list(held):
            try:
                release(slot)
            except Exception:
                pass
    if timing and result.decode_tokens:
        import sys
        both = result.forward_seconds + result.sample_seconds
        print(f"[MF_TIMING] over {result.decode_tokens} tokens: sample "
              f"{result.sample_seconds / result.decode_tokens * 1e3:6.2f} ms/tok "
              f"({100.0 * result.sample_seconds / both:4.1f}%), forward "
              f"{result.forward_seconds / result.decode_tokens * 1e3:6.2f} ms/tok "
              f"({100.0 * result.forward_seconds / both:4.1f}%)", file=sys.stderr)
    return result


def _decode_bound(engine, sampler, params, order, live, next_tok, windows, prompts, result, max_new, limit,
                  decide) -> Dict[int, int]:
    """Decodes the requests in `order` as one bound set until one of them ends, and returns the
    requests still alive.  The step after the one whose tokens the host is about to read is
    started first whenever no request can end by length in between: the device never waits
    for the host.  A request that ends on a stop token then has one more step in flight; its
    result is dropped, and what that step wrote into the cache goes with the sequence."""
    cap = max(min(len(prompts[r]) + max_new, limit) for r in order)
    session = engine.decode_session(len(order), cap, sampler)
    session.bind([live[r] for r in order], [next_tok[r] for r in order], order,
                 [len(result.tokens[r]) for r in order], sampler=sampler)
    if params.has_penalties:
        session.set_windows([windows[r] for r in order])
    slots = dict(live)
    alive = set(order)
    held = {r: engine.length(slots[r]) for r in order}      # tokens in the cache after the step taken last

    def take(tokens) -> None:
        """The tokens of one step, for the requests that had not ended before it."""
        now: Dict[int, int] = {}
        for r, tok in zip(order, tokens):
            if r not in alive:
                continue
            held[r] += 1
            result.decode_tokens += 1
            windows[r] = (windows[r] + [tok])[-REPEAT_LAST_N:]
            decide(r, tok, slots[r], now, held[r])
        alive.intersection_update(now)

    try:
        _run_bound(session, order, result, max_new, limit, held, alive, take)
    except BaseException:
        session.abandon()
        raise
    return {r: slots[r] for r in order if r in alive}


def _run_bound(session, order, result, max_new, limit, held, alive, take) -> None:
    pending = session.launch()
    while True:
        ahead = None
        # `pending` has been launched and not taken: it will bring every request to
        # len + 1 tokens and held + 1 positions; one more step must be allowed after that
        if all(len(result.tokens[r]) + 1 < max_new and held[r] + 2 <= limit for r in order):
            ahead = session.launch()
        take(session.collect(pending))
        if ahead is None:
            break
        if len(alive) < len(order):       # somebody ended: finish the step in flight, then rebind
            take(session.collect(ahead))
            break
        pending = ahead


def _sample(sampler: Sampler, logits: torch.Tensor, keys: Sequence[int], steps: Sequence[int],
            windows: Sequence[Sequence[int]], device) -> List[int]:
    n = logits.shape[0]
    out = torch.empty(n, dtype=torch.int32, device=device)
    prev = n_prev = None
    if sampler.params.has_penalties:
        flat = torch.zeros((n, REPEAT_LAST_N), dtype=torch.int32)
        for i, w in enumerate(windows):
            w = list(w)[-REPEAT_LAST_N:]
            if w:
                flat[i, :len(w)] = torch.tensor(w, dtype=torch.int32)
        prev = flat.to(device)
        n_prev = torch.tensor([min(len(w), REPEAT_LAST_N) for w in windows], dtype=torch.int32, device=device)
    sampler(logits, torch.tensor(sampler.streams(keys), dtype=torch.int64, device=device),
            torch.tensor(list(steps), dtype=torch.int32, device=device), out, prev, n_prev)
    return out.cpu().tolist()

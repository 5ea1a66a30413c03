"""The generation loop's decisions, without a GPU: a scripted engine that spikes a
programmed token and records what it is fed (the reference's MockEngine,
src/conversation.rs:586-613 of yusiwen/minfer), and the real engine on the CPU through the
plain kernels."""
import numpy as np
import pytest
import torch

import plain_ops
import plain_qwen2 as pq
from minfer_amd.engine.generate import generate, plan_batches
from minfer_amd.sampling import SamplingParams, uniform
from tiny import TINIES, random_tokens, write_tiny

GREEDY = SamplingParams.greedy()


class ScriptedEngine:
    """`script[request first token] = tokens it will produce`; logits spike the next one."""
    device = torch.device("cpu")

    def __init__(self, script, vocab=50, max_positions=1000, capacity=64 * 64, max_seqs=8):
        self.script, self.vocab_size = script, vocab
        self.max_positions, self._capacity, self.max_seqs = max_positions, capacity, max_seqs
        self.calls, self.seqs, self.free, self.ended = [], {}, list(range(max_seqs - 1, -1, -1)), []

    def capacity_tokens(self):
        return self._capacity

    def stop_tokens(self):
        return (0,)

    def new_sequence(self):
        s = self.free.pop()
        self.seqs[s] = []
        return s

    def end_sequence(self, slot):
        self.ended.append(slot)
        del self.seqs[slot]
        self.free.append(slot)

    def length(self, slot):
        return len(self.seqs[slot])

    def step(self, slots, tokens, want="last"):
        assert want == "last"
        self.calls.append((list(slots), [list(t) for t in tokens], [len(self.seqs[s]) for s in slots]))
        out = torch.full((len(slots), self.vocab_size), -5.0)
        for i, (s, t) in enumerate(zip(slots, tokens)):
            first = not self.seqs[s]
            self.seqs[s].extend(t)
            if first:
                self.seqs[s + 1000] = (self.seqs[s][0], len(t))
            key, plen = self.seqs[s + 1000]
            produced = len(self.seqs[s]) - plen
            plan = self.script[key]
            out[i, plan[produced] if produced < len(plan) else 0] = 5.0
        return out

    def end_bookkeeping(self):
        return {k: v for k, v in self.seqs.items() if k < 1000}


@pytest.fixture(autouse=True)
def cpu_kernels(monkeypatch):
    plain_ops.install(monkeypatch)


def test_stop_token_ends_only_its_own_sequence_and_is_not_emitted():
    eng = ScriptedEngine({10: [5, 6, 0, 9], 20: [7, 8, 9, 11, 12, 0]})
    res = generate(eng, [[10, 1, 2], [20, 3]], GREEDY, max_new=10, use_graph=False)
    assert res.tokens == [[5, 6], [7, 8, 9, 11, 12]] and res.finish_reasons == ["stop", "stop"]
    # prompts in one step at positions 0; then one token each, the sampled one, at the next position
    assert eng.calls[0] == ([0, 1], [[10, 1, 2], [20, 3]], [0, 0])
    assert eng.calls[1] == ([0, 1], [[5], [7]], [3, 2])
    assert eng.calls[2] == ([0, 1], [[6], [8]], [4, 3])
    # request 0 stopped: the stop token is not fed, the other sequence goes on alone
    assert eng.calls[3] == ([1], [[9]], [4])
    assert all(0 not in t for call in eng.calls[1:] for t in call[1])
    assert eng.end_bookkeeping() == {} and sorted(eng.ended) == [0, 1]


def test_max_new_is_honoured_without_a_wasted_forward():
    eng = ScriptedEngine({10: [5, 6, 7, 8, 9]})
    res = generate(eng, [[10]], GREEDY, max_new=3, use_graph=False)
    assert res.tokens == [[5, 6, 7]] and res.finish_reasons == ["length"]
    assert len(eng.calls) == 3                 # prompt, then 5 and 6 are fed; 7 is not
    assert res.decode_tokens == 2 and res.prefill_tokens == 1
    assert generate(eng, [[10]], GREEDY, max_new=0, use_graph=False).tokens == [[]]


def test_first_sampled_token_may_be_the_stop():
    eng = ScriptedEngine({10: [0], 20: [4, 0]})
    res = generate(eng, [[10], [20]], GREEDY, max_new=5, use_graph=False)
    assert res.tokens == [[], [4]] and res.finish_reasons == ["stop", "stop"]
    assert eng.calls[1][0] == [1]


def test_context_full_stops_cleanly():
    eng = ScriptedEngine({10: [5] * 50}, max_positions=6)
    res = generate(eng, [[10, 1, 2, 3]], GREEDY, max_new=40, use_graph=False)
    # positions 0..5: 4 prompt tokens + 2 fed tokens; the third sampled token is emitted, not fed
    assert res.tokens == [[5, 5, 5]] and res.finish_reasons == ["length"]
    assert [c[2] for c in eng.calls] == [[0], [4], [5]]
    res = generate(eng, [[10, 1, 2, 3]], GREEDY, max_new=40, use_graph=False, n_ctx=5)
    assert res.tokens == [[5, 5]]


def test_requests_run_in_batches_one_after_another_and_slots_are_reused():
    script = {10 + i: [5 + i] * (2 + i) + [0] for i in range(5)}
    eng = ScriptedEngine(script, capacity=64 * 2, max_seqs=2)
    res = generate(eng, [[10 + i] for i in range(5)], GREEDY, max_new=20, use_graph=False)
    assert res.batches == [[0, 1], [2, 3], [4]]
    assert res.tokens == [[5 + i] * (2 + i) for i in range(5)]
    assert sorted(set(s for c in eng.calls for s in c[0])) == [0, 1]     # two slots, used again


def test_plan_batches():
    assert plan_batches([10, 10, 10], 20, 64 * 2, 8, 1000) == [[0, 1], [2]]
    assert plan_batches([10, 100, 10], 28, 64 * 3, 8, 1000) == [[0, 1], [2]]
    assert plan_batches([1] * 5, 1, 64 * 100, 2, 1000) == [[0, 1], [2, 3], [4]]
    with pytest.raises(ValueError, match="exceeds"):
        plan_batches([2000], 5, 64 * 100, 2, 1000)
    with pytest.raises(ValueError, match="cache holds"):
        plan_batches([500], 5, 64 * 2, 2, 1000)
    with pytest.raises(ValueError, match="empty"):
        plan_batches([0], 5, 64 * 2, 2, 1000)


def test_on_token_and_explicit_stop_tokens():
    eng = ScriptedEngine({10: [5, 6, 7, 0]})
    seen = []
    res = generate(eng, [[10]], GREEDY, max_new=10, stop_tokens=[7], use_graph=False,
                   on_token=lambda r, t: seen.append((r, t)))
    assert res.tokens == [[5, 6]] and seen == [(0, 5), (0, 6)]


@pytest.mark.parametrize("name,use_graph", [("A", False), ("A", True), ("B", False)])
def test_real_engine_on_cpu_matches_plain_generation(tmp_path, name, use_graph):
    """Unequal prompts in one batch, sampling with the reference's default options, against
    the plain model sampled with the plain sampler and the same uniforms."""
    from minfer_amd import LLM
    folder = write_tiny(tmp_path, name, seed=2)
    plain = pq.PlainQwen2.from_folder(folder)
    vocab = TINIES[name]["vocab_size"]
    llm = LLM(folder, dtype="float32", device="cpu", n_ctx=128, n_slots=3)
    prompts = [random_tokens(vocab, n, i) for i, n in enumerate((5, 9, 1, 13))]
    for temp in (0.0, 0.8):
        res = llm.generate(prompts, max_new=6, temp=temp, seed=11, stop_tokens=[], use_graph=use_graph)
        assert res.batches == [[0, 1, 2], [3]]
        for i, (p, got) in enumerate(zip(prompts, res.tokens)):
            seq, exp = list(p), []
            for s in range(6):
                logits = plain.forward(seq)[-1].astype(np.float32)
                t = pq.sample(logits, temp, uniform(11, i, s), 40, 0.95, 1.1, 0.0, 0.0, pq.recent_window(seq))
                exp.append(t)
                seq.append(t)
            assert got == exp, (temp, i)
    llm.engine.cache.check_invariants()
    assert not llm.engine.cache.live_slots()


def test_running_ahead_drops_what_follows_a_stop_and_respects_lengths(tmp_path):
    """The decode loop starts step n + 1 before it reads the tokens of step n.  A request that
    stops at step n then has a step in flight: nothing of it may show, the others must not
    notice, and no request may run past max_new or the context bound because of it."""
    from minfer_amd import LLM
    folder = write_tiny(tmp_path, "A", seed=4)
    vocab = TINIES["A"]["vocab_size"]
    llm = LLM(folder, dtype="float32", device="cpu", n_ctx=128, n_slots=4)
    prompts = [random_tokens(vocab, n, 10 + i) for i, n in enumerate((4, 7, 2, 9))]
    free = llm.generate(prompts, max_new=9, temp=0.0, stop_tokens=[]).tokens
    assert all(len(t) == 9 for t in free)
    # a token that request 1 produces in the middle and that the others do not produce earlier
    for k in range(2, 8):
        stop = free[1][k]
        first_hit = [t.index(stop) if stop in t else 99 for t in free]
        if first_hit[1] == k:
            break
    res = llm.generate(prompts, max_new=9, temp=0.0, stop_tokens=[stop])
    for i, got in enumerate(res.tokens):
        cut = first_hit[i]
        assert got == free[i][:cut], i
        assert res.finish_reasons[i] == ("stop" if cut < 9 else "length")
    llm.engine.cache.check_invariants()
    assert not llm.engine.cache.live_slots()
    # the context bound: prompt + generated never exceeds n_ctx, and every request gets all it may
    small = LLM(folder, dtype="float32", device="cpu", n_ctx=12, n_slots=4)
    res = small.generate(prompts, max_new=50, temp=0.0, stop_tokens=[])
    for p, got in zip(prompts, res.tokens):
        assert len(got) == 12 - len(p) + 1          # one from the prompt's step, one per free position
        assert got == llm.generate([p], max_new=len(got), temp=0.0, stop_tokens=[], use_graph=False).tokens[0]
    assert res.finish_reasons == ["length"] * 4
    assert not small.engine.cache.live_slots()


def test_step_errors_leave_the_cache_alone(tmp_path):
    from minfer_amd import LLM, StepError
    from minfer_amd.cache import CacheFull
    llm = LLM(write_tiny(tmp_path, "A", seed=0), dtype="float32", device="cpu", n_ctx=128, n_slots=2)
    s = llm.new_sequence()
    with pytest.raises(StepError, match="embedding id 512 >= vocab 512"):
        llm.step([s], [[1, 512]])
    with pytest.raises(StepError, match="no tokens"):
        llm.step([s], [[]])
    with pytest.raises(StepError, match="twice"):
        llm.step([s, s], [[1], [2]])
    with pytest.raises(StepError, match="not in use"):
        llm.step([7], [[1]])
    with pytest.raises(StepError, match="exceeds the model's 256 positions"):
        llm.step([s], [[1] * 257])
    with pytest.raises(StepError, match="outside"):
        llm.step([s], [[1, 2]], [[2]])
    assert llm.engine.length(s) == 0 and llm.engine.cache.free_tokens() == 256
    t = llm.new_sequence()
    llm.step([s], [[1] * 200])
    with pytest.raises(CacheFull):
        llm.step([t], [[1] * 100])
    assert llm.engine.length(t) == 0
    llm.engine.cache.check_invariants()


def test_an_error_in_the_middle_of_a_batch_leaves_no_slot_taken(tmp_path):
    """A step that raises, or an `on_token` that raises, ends the call; every slot the call had
    taken is given back, so the engine is as free as before."""
    class Failing(ScriptedEngine):
        def step(self, slots, tokens, want="last"):
            if len(self.calls) == 2:
                raise RuntimeError("scripted failure in the third step")
            return super().step(slots, tokens, want)
    eng = Failing({10: [5, 6, 7, 8, 9], 20: [7, 8, 9, 11, 12], 30: [1, 2, 3]}, max_seqs=2)
    with pytest.raises(RuntimeError, match="scripted failure"):
        generate(eng, [[10, 1], [20, 3], [30]], GREEDY, max_new=5, stop_tokens=[], use_graph=False)
    assert eng.end_bookkeeping() == {} and sorted(eng.free) == [0, 1]
    eng2 = ScriptedEngine({10: [5, 6, 7, 8, 9], 20: [7, 8, 9, 11, 12]})

    def boom(r, t):
        if t == 8:
            raise KeyError("callback")
    with pytest.raises(KeyError):
        generate(eng2, [[10, 1], [20, 3]], GREEDY, max_new=5, stop_tokens=[], use_graph=False, on_token=boom)
    assert eng2.end_bookkeeping() == {} and len(eng2.free) == 8
    # the real engine through the captured-step path of the loop (stand-in kernels on the host)
    from minfer_amd import LLM
    llm = LLM(write_tiny(tmp_path, "A", seed=2), dtype="float32", device="cpu", n_ctx=64, n_slots=2)
    count = []

    def third(r, t):
        count.append(t)
        if len(count) == 5:
            raise ValueError("stop here")
    with pytest.raises(ValueError, match="stop here"):
        llm.generate([[1, 2, 3], [4, 5]], max_new=6, temp=0.0, stop_tokens=[], on_token=third)
    assert not llm.engine.cache.live_slots()
    llm.engine.cache.check_invariants()
    assert llm.generate([[1, 2, 3], [4, 5]], max_new=3, temp=0.0, stop_tokens=[]).finish_reasons == ["length"] * 2


def test_stop_tokens_come_from_config_and_generation_config(tmp_path):
    """config.json's eos ids, joined by generation_config.json's (where a chat model lists its
    end-of-turn token); an explicit list replaces both."""
    import json
    from minfer_amd import LLM
    folder = write_tiny(tmp_path, "A", seed=2)                     # eos_token_id 7 in config.json
    llm = LLM(folder, dtype="float32", device="cpu", n_ctx=64, n_slots=1)
    assert llm.engine.stop_tokens() == (7,)
    with open(folder + "/generation_config.json", "w") as f:
        json.dump({"eos_token_id": [9, 7], "temperature": 0.7}, f)
    llm = LLM(folder, dtype="float32", device="cpu", n_ctx=64, n_slots=1)
    assert llm.engine.stop_tokens() == (7, 9)
    free = llm.generate([[1, 2, 3]], max_new=8, temp=0.0, stop_tokens=[]).tokens[0]
    with open(folder + "/generation_config.json", "w") as f:
        json.dump({"eos_token_id": free[2]}, f)
    llm = LLM(folder, dtype="float32", device="cpu", n_ctx=64, n_slots=1)
    res = llm.generate([[1, 2, 3]], max_new=8, temp=0.0)
    first = free.index(free[2])
    assert res.tokens[0] == free[:first] and res.finish_reasons == ["stop"]
    with open(folder + "/generation_config.json", "w") as f:
        json.dump({"eos_token_id": 99999}, f)
    from minfer_amd import ConfigError
    with pytest.raises(ConfigError, match="eos_token_id"):
        LLM(folder, dtype="float32", device="cpu", n_ctx=64, n_slots=1)

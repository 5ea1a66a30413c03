"""The engine against the plain implementation, in 32-bit and in bfloat16: each request
alone and whole; the last 32 tokens one by one; batches of unequal lengths whose shorter
requests end earlier, one batch after another so that slots are used again."""
import pytest

from plain_qwen2 import PlainQwen2
from replays import (batch_steps, chunk_steps, compare, plain_logits, requests_for, run_steps, tail_steps,
                     whole_steps)
from tiny import TINIES, TINY_LONG, write_tiny

pytestmark = pytest.mark.gpu

LENGTHS = {"A": (5, 9, 13, 70, 33), "B": (1, 7, 31, 64, 129, 40), "C": (3, 65, 18, 100)}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("models")
    return {name: write_tiny(tmp, name, seed=i) for i, name in enumerate(TINIES)}


@pytest.fixture(scope="module")
def plains(folders):
    return {name: PlainQwen2.from_folder(f) for name, f in folders.items()}


def engine_for(folder, dtype, max_tokens=2048):
    from minfer_amd import Engine, load_model
    return Engine(load_model(folder, dtype=dtype, device="cuda:0"), max_tokens=max_tokens, poison_cache=True)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(TINIES))
def test_three_replays_agree_with_plain(folders, plains, name, dtype):
    vocab = TINIES[name]["vocab_size"]
    reqs = requests_for(vocab, LENGTHS[name], seed=3)
    ref = plain_logits(plains[name], reqs)
    ids = list(reqs)
    eng = engine_for(folders[name], dtype, max_tokens=64 * 8)
    compare(run_steps(eng, whole_steps(reqs)), ref, dtype, f"tiny {name} whole")
    compare(run_steps(eng, tail_steps(reqs)), ref, dtype, f"tiny {name} last 32 one by one")
    batches = [ids[:3], ids[3:]] if len(ids) > 3 else [ids]
    compare(run_steps(eng, batch_steps(reqs, batches)), ref, dtype, f"tiny {name} unequal batches")
    compare(run_steps(eng, chunk_steps(reqs, batches)), ref, dtype, f"tiny {name} prompts in portions")
    compare(run_steps(eng, chunk_steps(reqs, [[r] for r in ids], sizes=(17,))), ref, dtype,
            f"tiny {name} prompts in portions of 17")
    assert not eng.cache.live_slots()


@pytest.mark.parametrize("stored", ["float32", "float16", "mixed"])
def test_other_storage_types_in_the_bfloat16_run(tmp_path, stored):
    """A tensor stored in 32 bits stays in 32 bits (and takes the 32-bit product with widened
    activations); float16 is widened exactly; a file may mix types."""
    import torch
    from safetensors.torch import load_file, save_file
    from minfer_amd import Engine, load_model
    folder = write_tiny(tmp_path, "A", seed=9)
    path = folder + "/model.safetensors"
    t = load_file(path)
    for n in list(t):
        if stored == "float32" or (stored == "mixed" and ("norm" in n or "o_proj" in n or "embed" in n)):
            t[n] = t[n].float()
        elif stored == "float16":
            t[n] = t[n].to(torch.float16)        # exact for these magnitudes? no: rounds differently
    save_file(t, path)
    plain = PlainQwen2.from_folder(folder)        # reads the file as it now is
    model = load_model(folder, dtype="bfloat16")
    want = torch.float32 if stored != "mixed" else torch.bfloat16
    assert model.blocks[0].feed_forward.down.weight.dtype == want
    assert model.blocks[0].mixer.o.weight.dtype == torch.float32
    eng = Engine(model, max_tokens=64 * 4, poison_cache=True)
    reqs = requests_for(512, (5, 70, 9), seed=4)
    ref = plain_logits(plain, reqs)
    compare(run_steps(eng, batch_steps(reqs, [list(reqs)])), ref, "bfloat16", f"stored {stored}")
    compare(run_steps(eng, tail_steps(reqs, tail=4)), ref, "bfloat16", f"stored {stored} one by one")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_truncate_then_feed_again_gives_the_same_rows(folders, plains, dtype):
    """A sequence rolled back to a shorter length and fed other tokens, then rolled back again and
    fed the first ones: the rows after each roll-back are those of a sequence that never held the
    dropped tokens, across a page edge and with pages given back in between."""
    import numpy as np
    name = "B"
    vocab = TINIES[name]["vocab_size"]
    reqs = requests_for(vocab, (150, 150), seed=11)
    a, b = reqs["r0"], reqs["r1"]
    eng = engine_for(folders[name], dtype, max_tokens=64 * 4)
    s = eng.new_sequence()
    first = eng.step([s], [a], "all").cpu().numpy()
    eng.truncate(s, 60)                                   # below the first page edge: two pages go back
    assert eng.length(s) == 60 and eng.cache.free_tokens() == 64 * 3
    mixed = a[:60] + b[60:140]
    second = eng.step([s], [mixed[60:]], "all").cpu().numpy()
    eng.truncate(s, 100)
    third = eng.step([s], [mixed[100:]], "all").cpu().numpy()
    eng.truncate(s, 60)
    again = eng.step([s], [a[60:]], "all").cpu().numpy()
    eng.end_sequence(s)
    eng.cache.check_invariants()
    ref_a, ref_m = plains[name].forward(a), plains[name].forward(mixed)
    rows = {("a", p): first[p] for p in range(150)}
    rows.update({("m", 60 + i): second[i] for i in range(80)})
    rows.update({("m2", 100 + i): third[i] for i in range(40)})
    rows.update({("a2", 60 + i): again[i] for i in range(90)})
    compare(rows, {"a": ref_a, "m": ref_m, "m2": ref_m, "a2": ref_a}, dtype, "truncate")
    if dtype == "float32":
        assert np.abs(again - first[60:]).max() < 2e-5
    with pytest.raises(Exception, match="truncate"):
        s2 = eng.new_sequence()
        eng.truncate(s2, 5)


def test_tiled_copies_of_the_weights_change_no_bit(folders):
    """A bfloat16 model keeps tiled second copies of its matrices for the steps of few tokens
    where the row length allows (a multiple of 32) and the device has room: the same logits, bit
    for bit, as without them, for prompts whole and for tokens one by one; none in 32 bits."""
    import numpy as np
    from minfer_amd import Engine, load_model
    from minfer_amd.kernels import tuning
    reqs = requests_for(TINIES["B"]["vocab_size"], (40, 7, 90), seed=8)
    out = {}
    for copies in (True, False):
        tuning.NO_DECODE_COPIES = not copies
        try:
            model = load_model(folders["B"], dtype="bfloat16", device="cuda:0")
        finally:
            tuning.NO_DECODE_COPIES = False
        assert (model.decode_copy_bytes > 0) == copies
        assert (model.blocks[0].mixer.qkv.tiled is not None) == copies
        assert model.blocks[0].feed_forward.down.tiled is None        # rows of 344: no multiple of 32
        eng = Engine(model, max_tokens=64 * 8, poison_cache=True)
        out[copies] = (run_steps(eng, tail_steps(reqs)), run_steps(eng, batch_steps(reqs, [list(reqs)])))
    for with_copies, without in zip(out[True], out[False]):
        assert with_copies.keys() == without.keys()
        for key in with_copies:
            assert np.array_equal(with_copies[key], without[key]), key
    assert load_model(folders["B"], dtype="float32", device="cuda:0").decode_copy_bytes == 0


def test_random_model_on_the_device_is_the_written_folder(tmp_path):
    """`write_random_model` + `load_model` and `random_model` give the same tensors for the same
    configuration and seed, in both run types: one stream of random numbers, host and device."""
    import torch
    from minfer_amd import config_from_dict, load_model, random_model, write_random_model
    for name, seed in (("A", 3), ("C", 12345678901)):
        cfg = config_from_dict(TINIES[name])
        folder = write_random_model(str(tmp_path / f"rw_{name}"), cfg, seed)
        for dtype in ("bfloat16", "float32"):
            loaded, made = load_model(folder, dtype=dtype), random_model(cfg, seed=seed, dtype=dtype)
            pairs = [(loaded.embedding.weight, made.embedding.weight), (loaded.head.weight, made.head.weight),
                     (loaded.final_norm.weight, made.final_norm.weight)]
            for lb, mb in zip(loaded.blocks, made.blocks):
                pairs += [(lb.mixer.qkv.weight, mb.mixer.qkv.weight), (lb.mixer.qkv.bias, mb.mixer.qkv.bias),
                          (lb.mixer.o.weight, mb.mixer.o.weight), (lb.feed_forward.down.weight, mb.feed_forward.down.weight),
                          (lb.mixer_norm.weight, mb.mixer_norm.weight)]
                if lb.feed_forward.fused is not None:
                    pairs.append((lb.feed_forward.fused, mb.feed_forward.fused))
                else:
                    pairs.append((lb.feed_forward.gate_up.weight, mb.feed_forward.gate_up.weight))
            for x, y in pairs:
                assert x.dtype == y.dtype and torch.equal(x, y)
            assert loaded.embedding.weight.float().std().item() == pytest.approx(cfg.initializer_range, rel=0.05)
    other = random_model(config_from_dict(TINIES["A"]), seed=4, dtype="bfloat16")
    assert not torch.equal(other.embedding.weight, load_model(str(tmp_path / "rw_A"), dtype="bfloat16").embedding.weight)


def test_sessions_and_memory_stay_flat_over_many_seeds(folders):
    """Twenty calls with twenty seeds: the seed is data of the captured step, so the engine keeps
    one decode session per batch size and the device memory in use does not grow."""
    import torch
    from minfer_amd import LLM
    from minfer_amd.engine.engine import MAX_SESSIONS
    llm = LLM(folders["A"], dtype="bfloat16", n_ctx=128, n_slots=2)
    prompts = [[5, 6, 7], [9, 10]]
    outs = set()
    sizes = []
    for seed in range(20):
        res = llm.generate(prompts, max_new=8, temp=0.9, seed=seed, stop_tokens=[])
        outs.add(tuple(map(tuple, res.tokens)))
        torch.cuda.synchronize()
        sizes.append((len(llm.engine._sessions), torch.cuda.memory_allocated()))
    assert len(outs) > 10, "different seeds give different tokens"
    assert sizes[-1][0] == sizes[2][0] <= 2, sizes
    assert sizes[-1][1] <= sizes[2][1], "allocated memory grew with the number of seeds"
    again = llm.generate(prompts, max_new=8, temp=0.9, seed=3, stop_tokens=[])
    assert tuple(map(tuple, again.tokens)) in outs
    # other options: other sessions, and never more than the bound
    for k in range(MAX_SESSIONS + 3):
        llm.generate(prompts, max_new=3, temp=0.5 + 0.01 * k, seed=1, stop_tokens=[])
    assert len(llm.engine._sessions) <= MAX_SESSIONS
    assert not llm.engine.cache.live_slots()


# ------------------------------------------------------------------ long prompts
@pytest.fixture(scope="module")
def long_model(tmp_path_factory):
    """Two layers with room for 4,096 positions.  The q and k matrices are scaled up so that the
    scores of a query spread over several units: a softmax over two thousand keys then rests on a
    few of them, wherever they lie, and a page of keys left out, read twice or taken from another
    sequence moves the logits by far more than the bounds (with the plain random weights every
    key weighs the same two-thousandth and such a fault hides in the rounding)."""
    import torch
    from safetensors.torch import load_file, save_file
    from minfer_amd import config_from_dict, write_random_model
    folder = write_random_model(str(tmp_path_factory.mktemp("long") / "m"), config_from_dict(TINY_LONG), seed=21)
    path = folder + "/model.safetensors"
    t = load_file(path)
    for name in list(t):
        if "q_proj.weight" in name or "k_proj.weight" in name:
            t[name] = (t[name].float() * 5.0).to(t[name].dtype)
    save_file(t, path)
    plain = PlainQwen2.from_folder(folder)
    reqs = requests_for(TINY_LONG["vocab_size"], (2100, 700, 1500), seed=22)
    ref = plain_logits(plain, reqs)
    # the construction does what it says: the last query's largest softmax weight in layer 0 is
    # far above 1 / keys
    import numpy as np
    import plain_qwen2 as pq
    toks = reqs["r0"]
    h = pq.embedding(plain.w["model.embed_tokens.weight"], toks)
    xn = pq.rms_norm(h, plain.w["model.layers.0.input_layernorm.weight"], plain.eps)
    pos = np.arange(len(toks))
    q = pq.rope_neox(pq.linear(xn[-1:], plain.w["model.layers.0.self_attn.q_proj.weight"],
                               plain.w["model.layers.0.self_attn.q_proj.bias"]), pos[-1:], plain.nh, plain.hd, plain.theta)
    k = pq.rope_neox(pq.linear(xn, plain.w["model.layers.0.self_attn.k_proj.weight"],
                               plain.w["model.layers.0.self_attn.k_proj.bias"]), pos, plain.nk, plain.hd, plain.theta)
    s = (k.reshape(len(toks), plain.nk, plain.hd)[:, 0] @ q.reshape(plain.nh, plain.hd)[0]) / np.sqrt(plain.hd)
    w = pq.softmax_rows(s[None])[0]
    assert w.max() > 20.0 / len(toks), f"scores are too flat for this test (largest weight {w.max():.4f})"
    return folder, reqs, ref


def _wanted(n_new: int, first: int = 0):
    """The last 16 rows of a step's new tokens and a few in the middle, as offsets."""
    mid = [o for o in (0, 1, 63, 64, 65, n_new // 3, n_new // 2, n_new // 2 + 1) if 0 <= o < n_new - 16]
    return sorted(set(mid + list(range(max(0, n_new - 16), n_new))))


def _step_rows(eng, slots, ids, chunks, starts, rows):
    """One engine step through its three stages (so the test can look at the step's context);
    logits of the wanted offsets into `rows` as (request, position)."""
    want = [_wanted(len(c)) for c in chunks]
    ctx = eng.build_context([slots[r] for r in ids], chunks, want)
    logits = eng.model.forward(ctx).cpu().numpy()
    eng.cache.commit(ctx.new_lengths)
    eng.cache.check_invariants()
    r = 0
    for rid, offs, start in zip(ids, want, starts):
        for o in offs:
            rows[(rid, start + o)] = logits[r]
            r += 1
    assert r == logits.shape[0]
    return ctx


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_prompts_agree_with_plain(long_model, dtype):
    """Prompts of 2,100, 700 and 1,500 tokens in one step, and then, on the same engine (pages
    used again, poisoned in between), 64 new tokens of each on some 2,000, 600 and 1,400 cached
    ones: the case in which the prompt attention shares a block of queries' pages between several
    workgroups.  Logits of the last 16 rows of every portion and of some in the middle against the
    plain implementation."""
    folder, reqs, ref = long_model
    ids = list(reqs)
    eng = engine_for(folder, dtype, max_tokens=64 * 70)
    # all three whole, in one step
    slots = {r: eng.new_sequence() for r in ids}
    rows = {}
    _step_rows(eng, slots, ids, [reqs[r] for r in ids], [0, 0, 0], rows)
    for r in ids:
        eng.end_sequence(slots[r])
    compare(rows, ref, dtype, "long prompts, one step", layers=2)
    # all but the last 100 tokens, then 64 on top of them, then the rest
    slots = {r: eng.new_sequence() for r in ids}
    rows = {}
    heads = [len(reqs[r]) - 100 for r in ids]
    _step_rows(eng, slots, ids, [reqs[r][:n] for r, n in zip(ids, heads)], [0, 0, 0], rows)
    ctx = _step_rows(eng, slots, ids, [reqs[r][n:n + 64] for r, n in zip(ids, heads)], heads, rows)
    if dtype == "bfloat16":
        shared = [v for k, v in ctx._memo.items() if k[0] == "shared_query_tiles"]
        assert shared and shared[0] is not None, "this step was meant to share its query blocks' pages"
        assert shared[0][4] > 1
    _step_rows(eng, slots, ids, [reqs[r][n + 64:] for r, n in zip(ids, heads)], [n + 64 for n in heads], rows)
    for r in ids:
        eng.end_sequence(slots[r])
    compare(rows, ref, dtype, "long prompts, 64 tokens on a long cache", layers=2)
    assert not eng.cache.live_slots()

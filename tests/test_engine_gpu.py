"""The engine against the plain implementation, in 32-bit and in bfloat16: each request
alone and whole; the last 32 tokens one by one; batches of unequal lengths whose shorter
requests end earlier, one batch after another so that slots are used again."""
import pytest

from plain_qwen2 import PlainQwen2
from replays import batch_steps, compare, plain_logits, requests_for, run_steps, tail_steps, whole_steps
from tiny import TINIES, write_tiny

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

"""One layer at the widths of Qwen2.5-7B (hidden 3584, 28 heads over 4 kv heads of 128,
feed-forward 18944, vocabulary 152064) with random weights: 32-bit logits against the plain
implementation under the three ways of cutting, and bfloat16 within its tolerance.  The
sums here are as long as in the full model (18944 terms in the down product)."""
import numpy as np
import pytest

from plain_qwen2 import PlainQwen2
from replays import batch_steps, compare, plain_logits, requests_for, run_steps, tail_steps, whole_steps

pytestmark = pytest.mark.gpu

SHAPE_7B_ONE_LAYER = dict(
    architectures=["Qwen2ForCausalLM"], model_type="qwen2", hidden_act="silu",
    num_hidden_layers=1, hidden_size=3584, num_attention_heads=28, num_key_value_heads=4,
    intermediate_size=18944, vocab_size=152064, rope_theta=1000000.0, rms_norm_eps=1e-6,
    max_position_embeddings=32768, tie_word_embeddings=True, use_sliding_window=False)


@pytest.fixture(scope="module")
def folder(tmp_path_factory):
    from minfer_amd import config_from_dict, write_random_model
    return write_random_model(str(tmp_path_factory.mktemp("shape7b") / "m"), config_from_dict(SHAPE_7B_ONE_LAYER), seed=5)


@pytest.fixture(scope="module")
def reference(folder):
    plain = PlainQwen2.from_folder(folder, dtype=np.float64)
    reqs = requests_for(152064, (3, 20, 9, 37), seed=6)
    return reqs, plain_logits(plain, reqs)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_one_layer_at_7b_widths(folder, reference, dtype):
    from minfer_amd import Engine, load_model
    reqs, ref = reference
    ids = list(reqs)
    eng = Engine(load_model(folder, dtype=dtype), max_tokens=64 * 4, poison_cache=True)
    worst = max(compare(run_steps(eng, whole_steps(reqs)), ref, dtype, "7B widths whole"),
                compare(run_steps(eng, tail_steps(reqs, tail=8)), ref, dtype, "7B widths one by one"),
                compare(run_steps(eng, batch_steps(reqs, [ids[:3], ids[3:]])), ref, dtype, "7B widths batches"))
    print(f"{dtype}: worst abs err {worst:.3e}")


def test_batch_of_twenty_at_7b_widths(folder):
    """Twenty short requests in one batch: the prompts' step has some 60 rows and the decode steps
    20 down to 1, so the products run in the kernels for 17 to 64 rows (one block per CU over the
    whole of K for gate|up and the head, K split for the others) and then in those for at most 16."""
    from minfer_amd import Engine, load_model
    plain = PlainQwen2.from_folder(folder, dtype=np.float64)
    reqs = requests_for(152064, [3 + (i * 5) % 7 for i in range(20)], seed=8)
    ref = plain_logits(plain, reqs)
    eng = Engine(load_model(folder, dtype="bfloat16"), max_tokens=64 * 20, poison_cache=True)
    steps = batch_steps(reqs, [list(reqs)], prompt_frac=0.5)
    assert 17 <= sum(len(e["tokens"]) for e in steps[0]["entries"]) <= 64 and len(steps[1]["entries"]) > 16
    worst = compare(run_steps(eng, steps), ref, "bfloat16", "7B widths, batch of 20")
    print(f"worst abs err {worst:.3e}")


SHAPE_72B_ONE_LAYER = dict(
    architectures=["Qwen2ForCausalLM"], model_type="qwen2", hidden_act="silu",
    num_hidden_layers=1, hidden_size=8192, num_attention_heads=64, num_key_value_heads=8,
    intermediate_size=29568, vocab_size=3000, rope_theta=1000000.0, rms_norm_eps=1e-5,
    max_position_embeddings=32768, tie_word_embeddings=False, use_sliding_window=False)


def test_one_layer_at_72b_widths_in_32_bits(tmp_path_factory):
    """Hidden 8192 and feed-forward 29568 (a small vocabulary keeps the folder small) in the
    32-bit path: sums of up to 29568 terms, 64 heads over 8 kv heads, under the three ways of
    cutting.  (The bfloat16 kernels for K of 5120 and 8192 are checked one by one in
    test_kernels_gpu.py against references with the same rounded inputs; a bfloat16 run at
    these widths differs from the 64-bit plain implementation by about 1 % of the logits'
    standard deviation already at one layer, the branch outputs being hundreds of times larger
    than the embeddings with these random weights, which is more than the bound that the
    tiny configurations and the 7B widths are held to.)"""
    from minfer_amd import Engine, config_from_dict, load_model, write_random_model
    dtype = "float32"
    folder = write_random_model(str(tmp_path_factory.mktemp("shape72b") / "m"),
                                config_from_dict(SHAPE_72B_ONE_LAYER), seed=7)
    plain = PlainQwen2.from_folder(folder, dtype=np.float64)
    reqs = requests_for(3000, (3, 20, 9, 37), seed=9)
    ref = plain_logits(plain, reqs)
    ids = list(reqs)
    eng = Engine(load_model(folder, dtype=dtype), max_tokens=64 * 4, poison_cache=True)
    worst = max(compare(run_steps(eng, whole_steps(reqs)), ref, dtype, "72B widths whole"),
                compare(run_steps(eng, tail_steps(reqs, tail=8)), ref, dtype, "72B widths one by one"),
                compare(run_steps(eng, batch_steps(reqs, [ids[:3], ids[3:]])), ref, dtype, "72B widths batches"))
    print(f"{dtype}: worst abs err {worst:.3e}")

"""Tiny configurations of the architecture that differ in every size and option, and
helpers that write their model folders with random weights."""
from __future__ import annotations

import numpy as np

TINY_A = dict(
    architectures=["Qwen2ForCausalLM"], model_type="qwen2", hidden_act="silu",
    num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=2,
    intermediate_size=176, vocab_size=512, rope_theta=10000.0, rms_norm_eps=1e-6,
    max_position_embeddings=256, tie_word_embeddings=True, use_sliding_window=False,
    eos_token_id=7)

TINY_B = dict(
    architectures=["Qwen2ForCausalLM"], model_type="qwen2", hidden_act="silu",
    num_hidden_layers=3, hidden_size=128, num_attention_heads=4, num_key_value_heads=1,
    intermediate_size=344, vocab_size=1000, rope_theta=1000000.0, rms_norm_eps=1e-5,
    max_position_embeddings=512, tie_word_embeddings=False, use_sliding_window=False,
    eos_token_id=[3, 5])

# width that is not heads x head_dim, three kv groups of three heads, head_dim 48, an
# intermediate size and a vocabulary that are multiples of nothing useful
TINY_C = dict(
    architectures=["Qwen2ForCausalLM"], model_type="qwen2", hidden_act="silu",
    num_hidden_layers=1, hidden_size=200, num_attention_heads=9, num_key_value_heads=3,
    head_dim=48, intermediate_size=232, vocab_size=777, rope_theta=50000.0, rms_norm_eps=3e-6,
    max_position_embeddings=1024, tie_word_embeddings=False, initializer_range=0.05)

TINIES = {"A": TINY_A, "B": TINY_B, "C": TINY_C}

# for long prompts: room for 4,096 positions, two layers, three heads to a kv head
TINY_LONG = dict(
    architectures=["Qwen2ForCausalLM"], model_type="qwen2", hidden_act="silu",
    num_hidden_layers=2, hidden_size=192, num_attention_heads=6, num_key_value_heads=2,
    intermediate_size=272, vocab_size=600, rope_theta=1000000.0, rms_norm_eps=1e-6,
    max_position_embeddings=4096, tie_word_embeddings=False, use_sliding_window=False)


def write_tiny(tmp_path, name: str, seed: int = 0) -> str:
    from minfer_amd import config_from_dict, write_random_model
    folder = str(tmp_path / f"tiny_{name}_{seed}")
    write_random_model(folder, config_from_dict(TINIES[name]), seed)
    return folder


def random_tokens(vocab: int, length: int, seed: int):
    rng = np.random.default_rng(seed)
    return [int(t) for t in rng.integers(0, vocab, size=length)]

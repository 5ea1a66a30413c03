"""The size of the cache when none is given: what the device has free after the weights, less a
reserve, the largest step's activations and the sequences' fixed-size state, in whole pages (the
reference divides a given context over its slots, src/server/slot.rs:27-32 of yusiwen/minfer)."""
import pytest
import torch

from minfer_amd import config_from_dict
from minfer_amd.cache import PAGE, CacheError, KVRequest, StateRequest
from minfer_amd.engine.engine import (DEFAULT_STATE_SLOTS, RESERVE_BYTES_MIN, RESERVE_FRACTION, cache_bytes_per_token,
                                      plan_cache_tokens, state_bytes_per_sequence, tokens_that_fit)
from minfer_amd.engine.model import DecoderModel
from tiny import TINY_B

GIB = 1 << 30


def test_bytes_per_token_and_state():
    reqs = {0: KVRequest(4, 128), 1: KVRequest(4, 128), 2: StateRequest((3, 5)), 3: None,
            4: StateRequest((7,), torch.bfloat16)}
    assert cache_bytes_per_token(reqs, torch.bfloat16) == 2 * (2 * 4 * 128 * 2)       # the 7B shape: 2 KiB a layer
    assert cache_bytes_per_token(reqs, torch.float32) == 2 * (2 * 4 * 128 * 4)
    assert state_bytes_per_sequence(reqs) == 3 * 5 * 4 + 7 * 2


def test_plan_takes_reserve_step_and_state_off_and_rounds_to_pages():
    total = 288 * GIB
    reserve = int(RESERVE_FRACTION * total)
    assert reserve > RESERVE_BYTES_MIN
    per = 57344
    # exactly 1,000 pages and 5 bytes fit
    free = reserve + 1000 * PAGE * per + 5 + 123456 + 777
    assert plan_cache_tokens(free, total, per, state_bytes=777, step_bytes=123456) == 1000 * PAGE
    assert plan_cache_tokens(free - 6, total, per, 777, 123456) == 999 * PAGE
    # a small device: the fixed minimum is the reserve
    assert plan_cache_tokens(RESERVE_BYTES_MIN + 3 * PAGE * per, 8 * GIB, per, 0, 0) == 3 * PAGE
    # state is taken off in full
    assert plan_cache_tokens(RESERVE_BYTES_MIN + 10 * PAGE * per, 8 * GIB, per, 4 * PAGE * per, 0) == 6 * PAGE


def test_no_room_is_an_error_that_says_why():
    with pytest.raises(CacheError, match="no room for a cache.*MiB free.*held back"):
        plan_cache_tokens(RESERVE_BYTES_MIN + 100, 8 * GIB, 57344, 0, 0)
    with pytest.raises(CacheError, match="per-sequence state"):
        plan_cache_tokens(3 * GIB, 8 * GIB, 1024, state_bytes=2 * GIB, step_bytes=0)


def test_tokens_that_fit_reads_the_model_and_the_memory_it_is_given():
    model = DecoderModel(config_from_dict(TINY_B).model_spec(), torch.bfloat16, "cpu")
    per = 3 * 2 * 1 * 32 * 2                      # three layers, K and V, one kv head of 32, two bytes
    assert cache_bytes_per_token(model.cache_requests(), torch.bfloat16) == per
    step = 8192 * 128 * 4 * 12
    total = 16 * GIB
    free = RESERVE_BYTES_MIN + step + 50 * PAGE * per
    assert tokens_that_fit(model, mem_info=lambda: (free, total)) == 50 * PAGE
    assert tokens_that_fit(model, max_step_tokens=0, mem_info=lambda: (free, total)) == (50 * PAGE * per + step) // per // PAGE * PAGE
    with pytest.raises(CacheError):
        tokens_that_fit(model, mem_info=lambda: (RESERVE_BYTES_MIN, total))
    assert tokens_that_fit(model) == 1 << 30      # a model that is not on a GPU: no bound from here

    # a model whose mixers keep state: its slots' state comes off the budget
    class Stateful:
        rt, spec = model.rt, model.spec

        def cache_requests(self):
            return {0: KVRequest(1, 32), 1: StateRequest((1024, 256))}
    one = 1024 * 256 * 4
    per1 = 2 * 32 * 2
    free = RESERVE_BYTES_MIN + step + 8 * one + 20 * PAGE * per1
    assert tokens_that_fit(Stateful(), max_seqs=8, mem_info=lambda: (free, total)) == 20 * PAGE
    free = RESERVE_BYTES_MIN + step + DEFAULT_STATE_SLOTS * one + 20 * PAGE * per1
    assert tokens_that_fit(Stateful(), mem_info=lambda: (free, total)) == 20 * PAGE

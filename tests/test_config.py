"""Typed configuration and the architecture registry."""
import json

import pytest

from minfer_amd import ConfigError, Qwen2Config, config_from_dict, load_config, registered_architectures
from tiny import TINY_A, TINY_B, TINY_C


def test_reads_every_key_and_defaults():
    c = config_from_dict(TINY_B)
    assert isinstance(c, Qwen2Config)
    assert (c.num_hidden_layers, c.hidden_size, c.num_attention_heads, c.num_key_value_heads) == (3, 128, 4, 1)
    assert c.head_dim == 32 and c.intermediate_size == 344 and c.vocab_size == 1000
    assert c.rope_theta == 1e6 and c.rms_norm_eps == 1e-5 and c.max_position_embeddings == 512
    assert c.tie_word_embeddings is False and c.eos_token_ids == (3, 5)
    d = config_from_dict(dict(architectures=["Qwen2ForCausalLM"], vocab_size=10, hidden_size=32,
                              intermediate_size=8, num_hidden_layers=1, num_attention_heads=2))
    # defaults of the reference: kv heads = heads, eps 1e-6, base 10000, context 32768
    assert d.num_key_value_heads == 2 and d.rms_norm_eps == 1e-6 and d.rope_theta == 10000.0
    assert d.max_position_embeddings == 32768 and d.eos_token_ids == () and d.tie_word_embeddings is False


def test_head_dim_may_differ_from_hidden_over_heads():
    c = config_from_dict(TINY_C)
    assert c.head_dim == 48 and c.hidden_size == 200 and c.num_attention_heads * c.head_dim != c.hidden_size
    spec = c.model_spec()
    assert spec.blocks[0].mixer.params["head_dim"] == 48
    assert spec.blocks[0].mixer.params["scale"] == pytest.approx(48 ** -0.5)


def test_round_trip_through_config_json(tmp_path):
    c = config_from_dict(TINY_A)
    (tmp_path / "config.json").write_text(json.dumps(c.to_dict()))
    assert load_config(str(tmp_path)) == c
    assert load_config(str(tmp_path / "config.json")) == c


@pytest.mark.parametrize("change,needle", [
    (dict(architectures=["LlamaForCausalLM"]), "Unsupported architecture: 'LlamaForCausalLM'"),
    (dict(architectures=[]), "architectures"),
    (dict(hidden_size=None), "hidden_size"),
    (dict(num_attention_heads=3, hidden_size=64), "not a multiple of"),
    (dict(num_key_value_heads=3), "num_key_value_heads"),
    (dict(head_dim=15), "odd"),
    (dict(use_sliding_window=True), "use_sliding_window"),
    (dict(rope_scaling={"type": "yarn", "factor": 4.0}), "rope_scaling"),
    (dict(hidden_act="gelu"), "hidden_act"),
    (dict(vocab_size=0), "vocab_size"),
    (dict(rms_norm_eps="tiny"), "rms_norm_eps"),
    (dict(tie_word_embeddings="yes"), "tie_word_embeddings"),
    (dict(eos_token_id=99999), "eos_token_id"),
    (dict(layer_types=["full_attention", "sliding_attention"]), "layer_types"),
])
def test_rejections_name_the_key(change, needle):
    raw = dict(TINY_A)
    raw.update(change)
    with pytest.raises(ConfigError) as e:
        config_from_dict(raw)
    assert needle in str(e.value)


def test_unknown_architecture_lists_registered_names():
    with pytest.raises(ConfigError) as e:
        config_from_dict(dict(TINY_A, architectures=["Nope"]))
    assert "Qwen2ForCausalLM" in str(e.value)
    assert "Qwen2ForCausalLM" in registered_architectures()


def test_missing_config_file(tmp_path):
    with pytest.raises(ConfigError):
        load_config(str(tmp_path))
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(ConfigError):
        load_config(str(tmp_path))


def test_model_spec_is_data():
    spec = config_from_dict(TINY_B).model_spec()
    assert len(spec.blocks) == 3 and [e.block for e in spec.schedule] == [0, 1, 2]
    assert [e.cache for e in spec.schedule] == [0, 1, 2] and all(e.writes_cache for e in spec.schedule)
    assert spec.head_name == "lm_head.weight" and config_from_dict(TINY_A).model_spec().head_name is None
    b = spec.blocks[1]
    assert b.prefix == "model.layers.1." and b.mixer.kind == "gqa_attention" and b.feed_forward.kind == "swiglu"
    assert b.mixer_norm.params["eps"] == 1e-5 and b.mixer.params["position"].params["theta"] == 1e6
    assert spec.stop_tokens == (3, 5)


def test_schedule_is_checked():
    from minfer_amd.parts.spec import ModelSpec, RunEntry
    spec = config_from_dict(TINY_A).model_spec()
    kw = {f: getattr(spec, f) for f in spec.__dataclass_fields__}
    with pytest.raises(ValueError, match="written by"):
        ModelSpec(**dict(kw, schedule=(RunEntry(0, 0), RunEntry(1, 0))))
    with pytest.raises(ValueError, match="before any"):
        ModelSpec(**dict(kw, schedule=(RunEntry(0, 1, writes_cache=False), RunEntry(1, 1))))
    with pytest.raises(ValueError, match="names block"):
        ModelSpec(**dict(kw, schedule=(RunEntry(5, 0),)))
    ok = ModelSpec(**dict(kw, schedule=(RunEntry(0, 0), RunEntry(1, 1), RunEntry(0, 2), RunEntry(1, 1, writes_cache=False))))
    assert len(ok.schedule) == 4

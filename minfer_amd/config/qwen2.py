"""Qwen2 dense decoder: its config.json keys as a typed configuration, and the model
description built from them.

Hyper-parameters and their defaults follow `HParams` and `hparams_from_gguf` of
yusiwen/minfer (src/models/qwen2/loader.rs:11-29,97-147): kv heads default to the number
of heads, eps to 1e-6, the rotary base to 10000, the context to 32768; the rotary style is
the half-split one (loader.rs:144) and the attention scale is 1/sqrt(head_dim)
(loader.rs:36-38).  The reference has neither a sliding window nor frequency scaling, so
a config.json that asks for either is refused rather than run wrongly.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, asdict
from typing import Any, Dict, Tuple

from .base import ConfigError, KeyReader
from ..parts.spec import BlockSpec, ModelSpec, PartSpec, straight_schedule

ARCHITECTURE = "Qwen2ForCausalLM"


@dataclass(frozen=True)
class Qwen2Config:
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    max_position_embeddings: int
    rms_norm_eps: float
    rope_theta: float
    tie_word_embeddings: bool
    eos_token_ids: Tuple[int, ...]
    initializer_range: float

    architecture = ARCHITECTURE

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "Qwen2Config":
        r = KeyReader(raw)
        hidden = r.integer("hidden_size")
        heads = r.integer("num_attention_heads")
        kv_heads = r.integer("num_key_value_heads", default=heads)
        head_dim = r.integer("head_dim", default=None)
        if head_dim is None:
            if hidden % heads != 0:
                raise ConfigError(f"config.json: hidden_size {hidden} is not a multiple of "
                                  f"num_attention_heads {heads} and no head_dim is given")
            head_dim = hidden // heads
        if heads % kv_heads != 0:
            raise ConfigError(f"config.json: num_attention_heads {heads} is not a multiple of "
                              f"num_key_value_heads {kv_heads}")
        if head_dim % 2 != 0:
            raise ConfigError(f"config.json: head_dim {head_dim} is odd; the rotation pairs "
                              "element i with i + head_dim/2")
        act = r.string("hidden_act", default="silu")
        if act != "silu":
            raise ConfigError(f"config.json: hidden_act {act!r} is not supported; this "
                              "architecture's feed-forward uses 'silu'")
        if r.boolean("use_sliding_window", default=False):
            raise ConfigError("config.json: use_sliding_window=true is not supported: every "
                              "layer of this architecture attends to all earlier positions")
        layer_types = r.raw_value("layer_types")
        if layer_types is not None and any(t != "full_attention" for t in layer_types):
            raise ConfigError(f"config.json: layer_types {sorted(set(layer_types))} not "
                              "supported; only 'full_attention'")
        scaling = r.raw_value("rope_scaling")
        if scaling is not None:
            raise ConfigError(f"config.json: rope_scaling {scaling!r} is not supported; "
                              "rotation frequencies are unscaled")
        cfg = cls(
            vocab_size=r.integer("vocab_size"),
            hidden_size=hidden,
            intermediate_size=r.integer("intermediate_size"),
            num_hidden_layers=r.integer("num_hidden_layers"),
            num_attention_heads=heads,
            num_key_value_heads=kv_heads,
            head_dim=head_dim,
            max_position_embeddings=r.integer("max_position_embeddings", default=32768),
            rms_norm_eps=r.number("rms_norm_eps", default=1e-6),
            rope_theta=r.number("rope_theta", default=10000.0),
            tie_word_embeddings=r.boolean("tie_word_embeddings", default=False),
            eos_token_ids=r.token_ids("eos_token_id"),
            initializer_range=r.number("initializer_range", default=0.02),
        )
        for t in cfg.eos_token_ids:
            if t >= cfg.vocab_size:
                raise ConfigError(f"config.json: eos_token_id {t} >= vocab_size {cfg.vocab_size}")
        return cfg

    def to_dict(self) -> Dict[str, Any]:
        """A config.json that reads back to this configuration."""
        d = asdict(self)
        eos = d.pop("eos_token_ids")
        d["eos_token_id"] = list(eos) if len(eos) != 1 else eos[0]
        if not eos:
            d.pop("eos_token_id")
        d.update(architectures=[ARCHITECTURE], model_type="qwen2", hidden_act="silu",
                 use_sliding_window=False, rope_scaling=None, torch_dtype="bfloat16")
        return d

    # ---------------------------------------------------------------- description
    def model_spec(self) -> ModelSpec:
        """Every layer: RMSNorm -> grouped-query attention with biased q/k/v, unbiased o,
        half-split rotation -> add -> RMSNorm -> SwiGLU -> add
        (src/models/qwen2/graph.rs:59-177), then the final norm and the head."""
        norm = lambda name: PartSpec("rmsnorm", dict(
            size=self.hidden_size, eps=self.rms_norm_eps, weight=name))
        position = PartSpec("rope_neox", dict(
            head_dim=self.head_dim, theta=self.rope_theta,
            max_positions=self.max_position_embeddings))
        blocks = []
        for i in range(self.num_hidden_layers):
            mixer = PartSpec("gqa_attention", dict(
                hidden_size=self.hidden_size,
                n_heads=self.num_attention_heads,
                n_kv_heads=self.num_key_value_heads,
                head_dim=self.head_dim,
                scale=1.0 / math.sqrt(self.head_dim),
                window=None,
                qkv_bias=True, out_bias=False,
                position=position,
                q="self_attn.q_proj", k="self_attn.k_proj", v="self_attn.v_proj",
                o="self_attn.o_proj"))
            ffn = PartSpec("swiglu", dict(
                hidden_size=self.hidden_size, intermediate_size=self.intermediate_size,
                gate="mlp.gate_proj", up="mlp.up_proj", down="mlp.down_proj"))
            blocks.append(BlockSpec(
                kind="prenorm", prefix=f"model.layers.{i}.", mixer=mixer, feed_forward=ffn,
                mixer_norm=norm("input_layernorm.weight"),
                feed_forward_norm=norm("post_attention_layernorm.weight")))
        return ModelSpec(
            hidden_size=self.hidden_size, vocab_size=self.vocab_size,
            embedding_name="model.embed_tokens.weight",
            head_name=None if self.tie_word_embeddings else "lm_head.weight",
            final_norm=norm("model.norm.weight"),
            blocks=tuple(blocks), schedule=straight_schedule(len(blocks)),
            max_positions=self.max_position_embeddings,
            stop_tokens=self.eos_token_ids)

    def ignored_tensors(self) -> Tuple[str, ...]:
        """Tensors a file may hold that this configuration does not use: a stored copy of the
        head when it is tied to the embedding table."""
        return ("lm_head.weight",) if self.tie_word_embeddings else ()

    def random_init_std(self, tensor_name: str) -> float:
        """Standard deviation for random weights; norm gains are set to one instead."""
        return self.initializer_range

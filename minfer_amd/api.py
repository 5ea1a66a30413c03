"""Python entry point.

    from minfer_amd import LLM
    llm = LLM("model_dir", dtype="bfloat16", n_ctx=4096, n_slots=8)
    out = llm.generate([[1, 2, 3], [4, 5]], max_new=32, temp=0.0)
    out.tokens, out.finish_reasons, out.prefill_rate, out.decode_rate
    logits = llm.step(slots, token_lists, want="last")         # the step function itself

The reference has no Python API; option names, meanings and defaults are those of its
command line (`GenParams`, src/main.rs:42-70 of yusiwen/minfer).
"""
from __future__ import annotations

from typing import Any, Dict, Optional, Sequence, Union

from .cache.paged import PAGE
from .engine import Engine, GenerationResult, generate, load_model, random_model
from .engine.engine import cache_bytes_per_token, tokens_that_fit
from .sampling import SamplingParams


class LLM:
    def __init__(self, model: Optional[str] = None, *, config: Union[None, str, Dict[str, Any]] = None,
                 random_weights: bool = False, weight_seed: int = 0, dtype: str = "bfloat16",
                 n_ctx: int = 4096, n_slots: int = 8, max_tokens: Optional[int] = None,
                 device: str = "cuda:0"):
        """`model`: folder with config.json and model.safetensors.  With `random_weights`, the
        configuration comes from `config` (a dict or a config.json path) or from the folder's
        config.json, and weights are made on the device from `weight_seed`.  A sequence ends at
        `n_ctx` positions.  The cache holds `max_tokens` tokens; by default as many as `n_slots`
        sequences of `n_ctx` positions need, or what fits into the device memory that is free
        once the weights are loaded if that is less (`cache_plan` says which)."""
        if random_weights:
            from .config.base import read_config_json
            src = config if config is not None else model
            if src is None:
                raise ValueError("random_weights needs a configuration (config=... or a model folder)")
            raw = src if isinstance(src, dict) else read_config_json(src)
            self.model = random_model(raw, seed=weight_seed, dtype=dtype, device=device)
        else:
            if model is None:
                raise ValueError("a model folder is needed (or random_weights=True with a config)")
            self.model = load_model(model, dtype=dtype, device=device)
        self.config = self.model.config
        self.n_ctx = min(int(n_ctx), self.model.spec.max_positions)
        wanted = n_slots * ((self.n_ctx + PAGE - 1) // PAGE * PAGE)
        fits = None
        if max_tokens is None:
            fits = tokens_that_fit(self.model, max_seqs=n_slots)
            max_tokens = min(wanted, fits)
        self.engine = Engine(self.model, max_tokens=max_tokens, max_seqs=n_slots)
        per_token = cache_bytes_per_token(self.model.cache_requests(), self.model.rt.dtype)
        self.cache_plan = dict(tokens=self.engine.capacity_tokens(), slots=n_slots, context=self.n_ctx,
                               bytes=self.engine.capacity_tokens() * per_token, bytes_per_token=per_token,
                               fits=fits, limited_by_memory=fits is not None and fits < wanted)

    @classmethod
    def from_pretrained(cls, folder: str, **kw) -> "LLM":
        return cls(folder, **kw)

    @classmethod
    def random(cls, config: Union[str, Dict[str, Any]], seed: int = 0, **kw) -> "LLM":
        return cls(config=config, random_weights=True, weight_seed=seed, **kw)

    # the step function and its sequences
    def new_sequence(self) -> int:
        return self.engine.new_sequence()

    def end_sequence(self, slot: int) -> None:
        self.engine.end_sequence(slot)

    def step(self, slots: Sequence[int], tokens: Sequence[Sequence[int]], want="last"):
        return self.engine.step(slots, tokens, want)

    def truncate(self, slot: int, length: int) -> None:
        """Rolls a sequence back to its first `length` tokens (see `Engine.truncate`)."""
        self.engine.truncate(slot, length)

    def generate(self, prompts: Sequence[Sequence[int]], max_new: int = 512, temp: float = 0.8,
                 top_k: int = 40, top_p: float = 0.95, repeat_penalty: float = 1.1,
                 frequency_penalty: float = 0.0, presence_penalty: float = 0.0, seed: int = 42,
                 stop_tokens: Optional[Sequence[int]] = None, use_graph: bool = True,
                 on_token=None) -> GenerationResult:
        """Token-id prompts in, generated token ids out (stop token not included)."""
        params = SamplingParams(temp=temp, top_k=top_k, top_p=top_p, repeat_penalty=repeat_penalty,
                                frequency_penalty=frequency_penalty, presence_penalty=presence_penalty,
                                seed=seed)
        return generate(self.engine, prompts, params, max_new=max_new, stop_tokens=stop_tokens,
                        use_graph=use_graph, on_token=on_token, n_ctx=self.n_ctx)

"""From a model folder (or a configuration and a seed) to a model with weights on the GPU.

The reference's `load_model` picks the model by the architecture string, reads typed
hyper-parameters, then tensors by name (src/models/mod.rs:74-87,
src/models/qwen2/loader.rs:215-350 of yusiwen/minfer).
"""
from __future__ import annotations

import json
import os
import warnings
from typing import Any, Dict, Tuple, Union

import torch

from ..config.base import ConfigError, read_config_json
from ..kernels import ops
from ..registry import config_from_dict
from ..weights.loader import FolderWeights
from ..weights.random_init import tensor_seed
from .model import DecoderModel

DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32,
          "fp32": torch.float32, torch.bfloat16: torch.bfloat16, torch.float32: torch.float32}


def run_dtype(name) -> torch.dtype:
    if name not in DTYPES:
        raise ValueError(f"dtype must be bfloat16 or float32, got {name!r}")
    return DTYPES[name]


def require_gpu(device) -> torch.device:
    device = torch.device(device)
    if device.type != "cuda" or not torch.cuda.is_available():
        raise RuntimeError("minfer_amd runs on an AMD GPU through its HIP kernels; no GPU is "
                           "visible and there is no CPU path")
    return device


def generation_stop_tokens(folder: str, vocab_size: int) -> Tuple[int, ...]:
    """The `eos_token_id` entries of the folder's generation_config.json (an id or a list of
    ids), if there is such a file.  A chat model's end-of-turn token is listed there and not in
    config.json; the reference stops on either (eos or <|im_end|>, src/main.rs:626-628 of
    yusiwen/minfer)."""
    path = os.path.join(folder, "generation_config.json")
    if not os.path.isfile(path):
        return ()
    try:
        with open(path) as f:
            raw = json.load(f)
    except (OSError, json.JSONDecodeError) as e:
        raise ConfigError(f"{path}: cannot be read as JSON ({e})") from None
    v = raw.get("eos_token_id") if isinstance(raw, dict) else None
    if v is None:
        return ()
    ids = v if isinstance(v, (list, tuple)) else [v]
    for t in ids:
        if isinstance(t, bool) or not isinstance(t, int) or not 0 <= t < vocab_size:
            raise ConfigError(f"{path}: 'eos_token_id' must hold token ids below {vocab_size}, found {v!r}")
    return tuple(int(t) for t in ids)


def load_model(folder: str, dtype="bfloat16", device="cuda:0") -> DecoderModel:
    """config.json picks the architecture; model.safetensors gives the tensors by name.  Stop
    tokens are config.json's, joined by generation_config.json's where the folder has one."""
    device = require_gpu(device)
    config = config_from_dict(read_config_json(folder))
    model = DecoderModel(config.model_spec(), run_dtype(dtype), device)
    model.config = config
    expected = model.expected_tensors()
    # tensors a file may hold without the model wanting them (a stored copy of a tied head)
    ignore = tuple(getattr(config, "ignored_tensors", lambda: ())())
    source = FolderWeights(folder, expected, model.rt.dtype, device, ignore=ignore)
    found = [n for n in ignore if n in source.files and n not in expected]
    if found:
        warnings.warn(f"{', '.join(found)} in the file is not used by this configuration and is ignored")
    model.load(source.get)
    spec_stops = tuple(model.spec.stop_tokens)
    extra = tuple(t for t in generation_stop_tokens(folder, model.spec.vocab_size) if t not in spec_stops)
    model.stop_tokens = spec_stops + extra
    return model


def random_model(config: Union[Dict[str, Any], Any], seed: int = 0, dtype="bfloat16",
                 device="cuda:0") -> DecoderModel:
    """Random weights made on the device (no file): the tensors that `write_random_model` writes
    for the same configuration and seed (in bfloat16) and `load_model` reads back, value for
    value: matrices, tables and biases N(0, std of the configuration) rounded to bfloat16, norm
    gains one; a tensor's values depend on (seed, its name, the index)."""
    device = require_gpu(device)
    if isinstance(config, dict):
        config = config_from_dict(config)
    dt = run_dtype(dtype)
    model = DecoderModel(config.model_spec(), dt, device)
    model.config = config
    expected = model.expected_tensors()

    def get(name: str) -> torch.Tensor:
        ts = expected[name]
        if ts.init == "ones":
            return torch.ones(ts.shape, dtype=dt, device=device)
        if ts.init == "zeros":
            return torch.zeros(ts.shape, dtype=dt, device=device)
        t = torch.empty(ts.shape, dtype=dt, device=device)
        ops.fill_normal(t, tensor_seed(seed, name), config.random_init_std(name), round_bf16=True)
        return t
    model.load(get)
    model.stop_tokens = tuple(model.spec.stop_tokens)
    return model

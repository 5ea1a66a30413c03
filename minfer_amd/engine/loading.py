"""From a model folder (or a configuration and a seed) to a model with weights on the GPU.

The reference's `load_model` picks the model by the architecture string, reads typed
hyper-parameters, then tensors by name (src/models/mod.rs:74-87,
src/models/qwen2/loader.rs:215-350 of yusiwen/minfer).
"""
from __future__ import annotations

import warnings
import zlib
from typing import Any, Dict, Union

import torch

from ..config.base import read_config_json
from ..kernels import ops
from ..registry import config_from_dict
from ..weights.loader import FolderWeights
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


def load_model(folder: str, dtype="bfloat16", device="cuda:0") -> DecoderModel:
    """config.json picks the architecture; model.safetensors gives the tensors by name."""
    device = require_gpu(device)
    config = config_from_dict(read_config_json(folder))
    model = DecoderModel(config.model_spec(), run_dtype(dtype), device)
    model.config = config
    expected = model.expected_tensors()
    ignore = ()
    if model.spec.head_name is None:
        ignore = ("lm_head.weight",)     # tied: a stored copy of the head is not used
    source = FolderWeights(folder, expected, model.rt.dtype, device, ignore=ignore)
    if any(n in source.files for n in ignore):
        warnings.warn("tie_word_embeddings is set: lm_head.weight in the file is ignored")
    model.load(source.get)
    return model


def random_model(config: Union[Dict[str, Any], Any], seed: int = 0, dtype="bfloat16",
                 device="cuda:0") -> DecoderModel:
    """Random weights made on the device (no file): matrices, tables and biases N(0, std of
    the configuration), norm gains one; a tensor's values depend on (seed, its name)."""
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
            return torch.ones(ts.shape, dtype=torch.float32, device=device)
        t = torch.empty(ts.shape, dtype=dt, device=device)
        ops.fill_normal(t, (int(seed) << 32) ^ zlib.crc32(name.encode()), config.random_init_std(name))
        return t
    model.load(get)
    return model

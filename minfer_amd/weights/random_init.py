"""Random-weights mode: writes a model folder (config.json, model.safetensors) from a
configuration and a seed.

The reference has no such mode (each of its model tests needs a real model file,
src/models/qwen2/graph.rs:455-462 of yusiwen/minfer).  Values depend only on
(seed, tensor name, index): matrices, tables and biases are N(0, std) with the
configuration's std, norm gains are one.  Tensors are written in bfloat16.
"""
from __future__ import annotations

import json
import os
import zlib
from typing import Callable, Dict

import numpy as np
import torch

from .loader import TensorSpec
from .safetensors_io import write_safetensors


def tensor_seed(seed: int, name: str):
    """Seed material of one tensor's stream."""
    return [int(seed) & 0xFFFFFFFF, zlib.crc32(name.encode("utf-8")), len(name)]


def random_tensor(seed: int, name: str, spec: TensorSpec, std: float,
                  dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    if spec.init == "ones":
        return torch.ones(spec.shape, dtype=dtype)
    if spec.init == "zeros":
        return torch.zeros(spec.shape, dtype=dtype)
    if spec.init != "normal":
        raise ValueError(f"{name}: unknown init {spec.init!r}")
    rng = np.random.Generator(np.random.PCG64(tensor_seed(seed, name)))
    values = rng.standard_normal(spec.shape, dtype=np.float32) * np.float32(std)
    return torch.from_numpy(values).to(dtype)


def write_random_model(folder: str, config, seed: int, dtype: torch.dtype = torch.bfloat16) -> str:
    """`config` is a registered configuration object (it has to_dict(), model_spec() and
    random_init_std(name)).  Returns the folder."""
    from ..engine.model import expected_tensors
    os.makedirs(folder, exist_ok=True)
    expected: Dict[str, TensorSpec] = expected_tensors(config.model_spec())
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(config.to_dict(), f, indent=1)
    order = list(expected)
    write_safetensors(
        os.path.join(folder, "model.safetensors"),
        [(n, tuple(expected[n].shape), dtype) for n in order],
        lambda n: random_tensor(seed, n, expected[n], config.random_init_std(n), dtype),
        metadata={"format": "pt", "seed": str(seed)})
    return folder

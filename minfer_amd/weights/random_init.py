"""Random-weights mode: writes a model folder (config.json, model.safetensors) from a
configuration and a seed.

The reference has no such mode (each of its model tests needs a real model file,
src/models/qwen2/graph.rs:455-462 of yusiwen/minfer).  Values depend only on
(seed, tensor name, index): matrices, tables and biases are N(0, std) with the
configuration's std, norm gains are one.  Tensors are written in bfloat16.

The numbers come from one counter-based generator that runs, bit for bit alike, on the host
(here) and on the GPU (`engine.loading.random_model`): csrc/random_normal.h.  A folder written
with a seed and a model made on the device with the same seed hold the same weights.
"""
from __future__ import annotations

import json
import os
import zlib
from typing import Dict

import torch

from .loader import TensorSpec
from .safetensors_io import write_safetensors


def tensor_seed(seed: int, name: str) -> int:
    """The 64-bit seed of one tensor's stream: the model's seed above, a checksum of the
    tensor's name below."""
    return ((int(seed) & 0xFFFFFFFF) << 32) ^ zlib.crc32(name.encode("utf-8"))


def random_tensor(seed: int, name: str, spec: TensorSpec, std: float,
                  dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """One tensor on the host.  A float32 tensor holds the unrounded float values; a bfloat16
    tensor the same values rounded to nearest even."""
    if spec.init == "ones":
        return torch.ones(spec.shape, dtype=dtype)
    if spec.init == "zeros":
        return torch.zeros(spec.shape, dtype=dtype)
    if spec.init != "normal":
        raise ValueError(f"{name}: unknown init {spec.init!r}")
    if dtype not in (torch.bfloat16, torch.float32):
        raise ValueError(f"{name}: random weights are written in bfloat16 or float32, not {dtype}")
    from ..kernels import ops
    out = torch.empty(spec.shape, dtype=dtype)
    ops.fill_normal_host(out, tensor_seed(seed, name), std, round_bf16=False)
    return out


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

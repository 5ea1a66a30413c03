"""Weights by tensor name, checked against what the model expects.

The reference looks every tensor up by exact name and treats most as optional until the
graph needs them (src/models/qwen2/loader.rs:242-320 of yusiwen/minfer); here the check is
strict and happens once: one error lists every missing tensor, every unexpected tensor and
every wrong shape.

Storage types: bfloat16 stays bfloat16; a tensor stored in 32 bits stays in 32 bits;
float16 is widened to float32 (exact); integer tables become int32.  The 32-bit run type
widens everything floating to float32 (exact for bfloat16 and float16).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Tuple

import torch

from .safetensors_io import SafetensorsError, open_model_files


class WeightError(ValueError):
    """The tensors of a model folder do not match the model."""


@dataclass(frozen=True)
class TensorSpec:
    """What a part expects of one tensor: its shape, and how random weights fill it
    ('normal': N(0, std) of the configuration; 'ones': norm gains)."""
    shape: Tuple[int, ...]
    init: str = "normal"


def storage_dtype(stored: torch.dtype, run_dtype: torch.dtype) -> torch.dtype:
    if not stored.is_floating_point:
        return torch.int32
    if run_dtype == torch.float32 or stored in (torch.float32, torch.float16, torch.float64):
        return torch.float32
    return torch.bfloat16


def check_against(expected: Dict[str, TensorSpec], found: Dict[str, Tuple[Tuple[int, ...], torch.dtype]],
                  where: str) -> None:
    """Raises one WeightError naming all missing, unexpected and mis-shaped tensors."""
    missing = sorted(n for n in expected if n not in found)
    unexpected = sorted(n for n in found if n not in expected)
    shapes = sorted(f"{n}: expected {list(expected[n].shape)}, found {list(found[n][0])}"
                    for n in expected if n in found and tuple(found[n][0]) != tuple(expected[n].shape))
    dtypes = sorted(f"{n}: {found[n][1]}" for n in expected
                    if n in found and not found[n][1].is_floating_point)
    if not (missing or unexpected or shapes or dtypes):
        return
    lines = [f"weights in {where} do not match the model:"]
    if missing:
        lines.append(f"  missing tensors ({len(missing)}): " + ", ".join(missing))
    if unexpected:
        lines.append(f"  unexpected tensors ({len(unexpected)}): " + ", ".join(unexpected))
    if shapes:
        lines.append(f"  wrong shapes ({len(shapes)}): " + "; ".join(shapes))
    if dtypes:
        lines.append(f"  not floating point ({len(dtypes)}): " + "; ".join(dtypes))
    raise WeightError("\n".join(lines))


class FolderWeights:
    """Weight source over a model folder.  `get(name)` returns the tensor on `device` in
    its storage type for `run_dtype`."""

    def __init__(self, folder: str, expected: Dict[str, TensorSpec], run_dtype: torch.dtype,
                 device, ignore=()):
        self.folder = folder
        try:
            self.files = open_model_files(folder)
        except SafetensorsError as e:
            raise WeightError(str(e)) from None
        found = {}
        for name, f in self.files.items():
            if name in ignore and name not in expected:
                continue
            dtype_name, shape, _, _ = f.entries[name]
            found[name] = (shape, _torch_dtype(dtype_name))
        check_against(expected, found, folder)
        self.run_dtype = run_dtype
        self.device = device

    def get(self, name: str) -> torch.Tensor:
        t = self.files[name].tensor(name)
        return t.to(device=self.device, dtype=storage_dtype(t.dtype, self.run_dtype))


def _torch_dtype(name: str) -> torch.dtype:
    from .safetensors_io import _DTYPES
    return _DTYPES[name][1]

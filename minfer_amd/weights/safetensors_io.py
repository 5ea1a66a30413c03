"""Reading and writing safetensors files without executing anything from them.

Layout: 8 bytes little-endian header length, a JSON header
`{name: {"dtype", "shape", "data_offsets": [begin, end]}, "__metadata__": {...}}`, then the
bytes.  Tensors are handed out as views of a memory map, so a file larger than host memory
can be walked tensor by tensor.  The reference indexes its model file by tensor name over
all parts of a split file and borrows slices of a memory map the same way
(src/models/qwen2/loader.rs:166-187,236-241 of yusiwen/minfer).
"""
from __future__ import annotations

import json
import os
import struct
from typing import Dict, Iterable, List, Tuple

import numpy as np
import torch

# name in the file -> (numpy dtype used for the view, torch dtype handed out)
_DTYPES = {
    "F64": (np.float64, torch.float64),
    "F32": (np.float32, torch.float32),
    "F16": (np.float16, torch.float16),
    "BF16": (np.int16, torch.bfloat16),
    "I64": (np.int64, torch.int64),
    "I32": (np.int32, torch.int32),
    "I16": (np.int16, torch.int16),
    "I8": (np.int8, torch.int8),
    "U8": (np.uint8, torch.uint8),
    "BOOL": (np.bool_, torch.bool),
}
_NAMES = {t: n for n, (_, t) in _DTYPES.items()}


class SafetensorsError(ValueError):
    pass


class SafetensorsFile:
    """One file: `entries[name] = (dtype name, shape, begin, end)`; `tensor(name)` returns
    a CPU tensor that views the map (copy-on-write, so nothing is ever written back)."""

    def __init__(self, path: str):
        self.path = path
        size = os.path.getsize(path)
        with open(path, "rb") as f:
            head = f.read(8)
            if len(head) != 8:
                raise SafetensorsError(f"{path}: shorter than a safetensors header")
            (n,) = struct.unpack("<Q", head)
            if n <= 0 or 8 + n > size:
                raise SafetensorsError(f"{path}: header length {n} does not fit the file ({size} bytes)")
            try:
                header = json.loads(f.read(n).decode("utf-8"))
            except (UnicodeDecodeError, json.JSONDecodeError) as e:
                raise SafetensorsError(f"{path}: header is not JSON ({e})") from None
        self.data_start = 8 + n
        self.metadata = header.pop("__metadata__", {}) or {}
        self.entries: Dict[str, Tuple[str, Tuple[int, ...], int, int]] = {}
        for name, info in header.items():
            try:
                dtype, shape = info["dtype"], tuple(int(s) for s in info["shape"])
                begin, end = (int(v) for v in info["data_offsets"])
            except (KeyError, TypeError, ValueError):
                raise SafetensorsError(f"{path}: malformed entry for tensor {name!r}") from None
            if dtype not in _DTYPES:
                raise SafetensorsError(f"{path}: tensor {name!r} has unsupported dtype {dtype}")
            count = int(np.prod(shape, dtype=np.int64)) if shape else 1
            if end - begin != count * np.dtype(_DTYPES[dtype][0]).itemsize or begin < 0 \
                    or self.data_start + end > size:
                raise SafetensorsError(f"{path}: tensor {name!r} offsets [{begin},{end}) do not "
                                       f"match dtype {dtype} and shape {list(shape)}")
            self.entries[name] = (dtype, shape, begin, end)
        self._map = None

    def names(self) -> List[str]:
        return list(self.entries)

    def tensor(self, name: str) -> torch.Tensor:
        dtype, shape, begin, end = self.entries[name]
        np_dtype, torch_dtype = _DTYPES[dtype]
        if self._map is None:
            self._map = np.memmap(self.path, dtype=np.uint8, mode="c")
        if end == begin:
            return torch.empty(shape, dtype=torch_dtype)
        raw = self._map[self.data_start + begin:self.data_start + end].view(np_dtype)
        t = torch.from_numpy(raw.reshape(shape))
        return t.view(torch.bfloat16) if dtype == "BF16" else t


def open_model_files(folder: str) -> Dict[str, SafetensorsFile]:
    """tensor name -> file holding it.  Reads `model.safetensors`, or the files named by
    `model.safetensors.index.json`'s weight_map."""
    single = os.path.join(folder, "model.safetensors")
    index = os.path.join(folder, "model.safetensors.index.json")
    by_name: Dict[str, SafetensorsFile] = {}
    if os.path.exists(single):
        f = SafetensorsFile(single)
        return {n: f for n in f.names()}
    if os.path.exists(index):
        with open(index) as fh:
            weight_map = json.load(fh).get("weight_map", {})
        files: Dict[str, SafetensorsFile] = {}
        for name, fname in weight_map.items():
            if fname not in files:
                files[fname] = SafetensorsFile(os.path.join(folder, fname))
            if name not in files[fname].entries:
                raise SafetensorsError(f"{index}: {name!r} is mapped to {fname}, which does not hold it")
            by_name[name] = files[fname]
        return by_name
    raise SafetensorsError(f"no model.safetensors (or model.safetensors.index.json) in {folder}")


def write_safetensors(path: str, tensors: Iterable[Tuple[str, Tuple[int, ...], torch.dtype]],
                      produce, metadata: Dict[str, str] = None) -> None:
    """Streams a file: `tensors` lists (name, shape, dtype) in file order and
    `produce(name)` returns each tensor when its turn comes, so only one is in memory."""
    tensors = list(tensors)
    header, offset = {}, 0
    for name, shape, dtype in tensors:
        if dtype not in _NAMES:
            raise SafetensorsError(f"cannot write dtype {dtype} for {name!r}")
        count = int(np.prod(shape, dtype=np.int64)) if len(shape) else 1
        nbytes = count * torch.empty((), dtype=dtype).element_size()
        header[name] = {"dtype": _NAMES[dtype], "shape": list(shape),
                        "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for name, shape, dtype in tensors:
            t = produce(name)
            if tuple(t.shape) != tuple(shape) or t.dtype != dtype:
                raise SafetensorsError(f"{name!r}: produced {tuple(t.shape)} {t.dtype}, "
                                       f"declared {tuple(shape)} {dtype}")
            t = t.contiguous().cpu()
            if t.dtype == torch.bfloat16:
                t = t.view(torch.int16)
            f.write(t.numpy().tobytes())
    os.replace(tmp, path)

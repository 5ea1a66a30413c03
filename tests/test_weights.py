"""Safetensors reading and writing, the one weight error, random-weights folders."""
import json
import os
import struct

import numpy as np
import pytest
import torch

from minfer_amd import WeightError, config_from_dict, write_random_model
from minfer_amd.engine.model import expected_tensors
from minfer_amd.weights import (FolderWeights, SafetensorsError, SafetensorsFile, TensorSpec, open_model_files,
                                random_tensor, storage_dtype, write_safetensors)
from tiny import TINY_A, TINY_B, write_tiny


def hand_built_file(path, tensors):
    """A safetensors file written byte by byte, independent of the product's writer."""
    header, blob = {}, b""
    for name, arr in tensors.items():
        code = {np.dtype("<f4"): "F32", np.dtype("<i8"): "I64", np.dtype("<f2"): "F16"}[arr.dtype]
        header[name] = {"dtype": code, "shape": list(arr.shape), "data_offsets": [len(blob), len(blob) + arr.nbytes]}
        blob += arr.tobytes()
    h = json.dumps(header).encode()
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(h)) + h + blob)


def test_reads_hand_built_file(tmp_path):
    a = np.arange(12, dtype="<f4").reshape(3, 4)
    b = np.array([5, -7], dtype="<i8")
    hand_built_file(tmp_path / "model.safetensors", {"a": a, "b": b})
    f = SafetensorsFile(str(tmp_path / "model.safetensors"))
    assert sorted(f.names()) == ["a", "b"]
    assert torch.equal(f.tensor("a"), torch.from_numpy(a)) and f.tensor("b").tolist() == [5, -7]


def test_writer_agrees_with_the_safetensors_library(tmp_path):
    from safetensors.torch import load_file
    t = {"x": torch.randn(5, 3).to(torch.bfloat16), "y": torch.arange(7, dtype=torch.float32)}
    write_safetensors(str(tmp_path / "w.safetensors"), [(n, tuple(v.shape), v.dtype) for n, v in t.items()],
                      lambda n: t[n], metadata={"format": "pt"})
    back = load_file(str(tmp_path / "w.safetensors"))
    assert all(torch.equal(back[n], t[n]) for n in t)
    mine = SafetensorsFile(str(tmp_path / "w.safetensors"))
    assert all(torch.equal(mine.tensor(n), t[n]) for n in t)


@pytest.mark.parametrize("blob", [b"", b"\x10\x00\x00", struct.pack("<Q", 1 << 40) + b"{}",
                                  struct.pack("<Q", 5) + b"notjs"])
def test_bad_headers_fail(tmp_path, blob):
    p = tmp_path / "model.safetensors"
    p.write_bytes(blob)
    with pytest.raises(SafetensorsError):
        SafetensorsFile(str(p))


def test_offsets_must_match_shape(tmp_path):
    h = json.dumps({"a": {"dtype": "F32", "shape": [4], "data_offsets": [0, 8]}}).encode()
    (tmp_path / "model.safetensors").write_bytes(struct.pack("<Q", len(h)) + h + b"\0" * 8)
    with pytest.raises(SafetensorsError, match="offsets"):
        SafetensorsFile(str(tmp_path / "model.safetensors"))


def test_random_folder_matches_expected_tensors(tmp_path):
    folder = write_tiny(tmp_path, "B", seed=4)
    cfg = config_from_dict(TINY_B)
    exp = expected_tensors(cfg.model_spec())
    files = open_model_files(folder)
    assert set(files) == set(exp)
    for n, spec in exp.items():
        t = files[n].tensor(n)
        assert tuple(t.shape) == spec.shape and t.dtype == torch.bfloat16
    assert "lm_head.weight" in exp and "model.layers.2.self_attn.q_proj.bias" in exp
    assert exp["model.layers.0.self_attn.k_proj.weight"].shape == (32, 128)
    gains = files["model.norm.weight"].tensor("model.norm.weight").float()
    assert torch.equal(gains, torch.ones_like(gains))
    w = files["model.embed_tokens.weight"].tensor("model.embed_tokens.weight").float()
    assert abs(w.mean().item()) < 1e-3 and abs(w.std().item() - 0.02) < 1e-3
    assert json.load(open(os.path.join(folder, "config.json")))["architectures"] == ["Qwen2ForCausalLM"]
    assert "lm_head.weight" not in expected_tensors(config_from_dict(TINY_A).model_spec())


def test_random_weights_depend_on_seed_and_name_only(tmp_path):
    a = write_tiny(tmp_path, "A", seed=1)
    b = write_tiny(tmp_path / "again", "A", seed=1) if (tmp_path / "again").mkdir() is None else None
    c = write_tiny(tmp_path, "A", seed=2)
    fa, fb, fc = (open_model_files(x) for x in (a, b, c))
    n = "model.layers.0.mlp.up_proj.weight"
    assert torch.equal(fa[n].tensor(n), fb[n].tensor(n))
    assert not torch.equal(fa[n].tensor(n), fc[n].tensor(n))
    spec = TensorSpec((4, 4))
    assert not torch.equal(random_tensor(1, "x", spec, 0.02), random_tensor(1, "y", spec, 0.02))


def edit_file(folder, edit):
    """Rewrites model.safetensors after `edit(dict of tensors)`."""
    from safetensors.torch import load_file, save_file
    p = os.path.join(folder, "model.safetensors")
    t = load_file(p)
    edit(t)
    save_file(t, p)


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    folder = write_tiny(tmp_path, "B", seed=0)

    def edit(t):
        del t["model.layers.1.mlp.down_proj.weight"]
        del t["model.layers.2.self_attn.v_proj.bias"]
        t["model.layers.0.extra.weight"] = torch.zeros(3)
        t["model.norm.weight"] = torch.ones(64, dtype=torch.bfloat16)
        t["model.layers.0.self_attn.q_proj.weight"] = torch.zeros(128, 64, dtype=torch.bfloat16)
    edit_file(folder, edit)
    exp = expected_tensors(config_from_dict(TINY_B).model_spec())
    with pytest.raises(WeightError) as e:
        FolderWeights(folder, exp, torch.bfloat16, "cpu")
    msg = str(e.value)
    for needle in ("missing tensors (2)", "model.layers.1.mlp.down_proj.weight", "model.layers.2.self_attn.v_proj.bias",
                   "unexpected tensors (1)", "model.layers.0.extra.weight", "wrong shapes (2)",
                   "model.norm.weight: expected [128], found [64]",
                   "model.layers.0.self_attn.q_proj.weight: expected [128, 128], found [128, 64]"):
        assert needle in msg, (needle, msg)


def test_missing_file_is_a_weight_error(tmp_path):
    with pytest.raises(WeightError, match="model.safetensors"):
        FolderWeights(str(tmp_path), {}, torch.bfloat16, "cpu")


def test_storage_types():
    bf, f32, f16 = torch.bfloat16, torch.float32, torch.float16
    assert storage_dtype(bf, bf) == bf           # bfloat16 stays
    assert storage_dtype(f32, bf) == f32         # a tensor stored in 32 bits stays so
    assert storage_dtype(f16, bf) == f32         # widened exactly
    assert storage_dtype(bf, f32) == f32 and storage_dtype(f32, f32) == f32
    assert storage_dtype(torch.int64, bf) == torch.int32


def test_loader_keeps_32_bit_tensors(tmp_path):
    folder = write_tiny(tmp_path, "A", seed=0)
    edit_file(folder, lambda t: t.update({"model.norm.weight": t["model.norm.weight"].float()}))
    exp = expected_tensors(config_from_dict(TINY_A).model_spec())
    src = FolderWeights(folder, exp, torch.bfloat16, "cpu")
    assert src.get("model.norm.weight").dtype == torch.float32
    assert src.get("model.embed_tokens.weight").dtype == torch.bfloat16
    assert FolderWeights(folder, exp, torch.float32, "cpu").get("model.embed_tokens.weight").dtype == torch.float32


def test_sharded_folder_with_index(tmp_path):
    from safetensors.torch import load_file, save_file
    folder = write_tiny(tmp_path, "A", seed=0)
    t = load_file(os.path.join(folder, "model.safetensors"))
    names = sorted(t)
    half = len(names) // 2
    save_file({n: t[n] for n in names[:half]}, os.path.join(folder, "model-00001-of-00002.safetensors"))
    save_file({n: t[n] for n in names[half:]}, os.path.join(folder, "model-00002-of-00002.safetensors"))
    os.remove(os.path.join(folder, "model.safetensors"))
    wm = {n: ("model-00001-of-00002.safetensors" if i < half else "model-00002-of-00002.safetensors")
          for i, n in enumerate(names)}
    json.dump({"weight_map": wm}, open(os.path.join(folder, "model.safetensors.index.json"), "w"))
    exp = expected_tensors(config_from_dict(TINY_A).model_spec())
    src = FolderWeights(folder, exp, torch.bfloat16, "cpu")
    assert torch.equal(src.get(names[-1]), t[names[-1]])

"""Reading and writing ``model.safetensors`` (single file or shards named by
``model.safetensors.index.json``) by tensor name."""

from __future__ import annotations

import json
import os

import torch
from safetensors import safe_open
from safetensors.torch import save_file


class WeightsError(RuntimeError):
    pass


def safetensors_files(folder: str) -> list[str]:
    index = os.path.join(folder, "model.safetensors.index.json")
    if os.path.isfile(index):
        with open(index) as f:
            names = sorted(set(json.load(f)["weight_map"].values()))
        return [os.path.join(folder, n) for n in names]
    single = os.path.join(folder, "model.safetensors")
    if os.path.isfile(single):
        return [single]
    raise WeightsError(f"no model.safetensors (or index) in {folder}")


def tensor_index(folder: str) -> dict[str, tuple[str, tuple[int, ...], str]]:
    """name -> (file, shape, dtype string) without reading any data."""
    out: dict[str, tuple[str, tuple[int, ...], str]] = {}
    for path in safetensors_files(folder):
        with safe_open(path, framework="pt") as f:
            for name in f.keys():
                sl = f.get_slice(name)
                out[name] = (path, tuple(sl.get_shape()), str(sl.get_dtype()))
    return out


def read_tensors(folder: str, names: list[str] | None = None) -> dict[str, torch.Tensor]:
    out: dict[str, torch.Tensor] = {}
    for path in safetensors_files(folder):
        with safe_open(path, framework="pt") as f:
            for name in f.keys():
                if names is None or name in names:
                    out[name] = f.get_tensor(name)
    return out


def read_safetensors_folder(folder: str) -> dict[str, torch.Tensor]:
    """Every tensor of a model folder on the CPU, as stored."""
    return read_tensors(folder)


def write_safetensors(folder: str, tensors: dict[str, torch.Tensor]) -> str:
    os.makedirs(folder, exist_ok=True)
    path = os.path.join(folder, "model.safetensors")
    save_file({k: v.contiguous() for k, v in tensors.items()}, path, metadata={"format": "pt"})
    return path

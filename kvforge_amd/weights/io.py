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
        paths = [os.path.join(folder, n) for n in names]
        gone = [n for n, path in zip(names, paths) if not os.path.isfile(path)]
        if gone:
            raise WeightsError(f"model.safetensors.index.json in {folder} names files that are "
                               f"not there: {gone}")
        return paths
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


def write_safetensors(folder: str, tensors: dict[str, torch.Tensor], shards: int = 1) -> str:
    """One ``model.safetensors``, or with ``shards > 1`` that many files of about equal size
    (tensors in name order) and the ``model.safetensors.index.json`` that names each tensor's
    file.  Returns the path of the file, or of the index."""
    os.makedirs(folder, exist_ok=True)
    single = os.path.join(folder, "model.safetensors")
    index = os.path.join(folder, "model.safetensors.index.json")
    if shards <= 1:
        save_file({k: v.contiguous() for k, v in tensors.items()}, single, metadata={"format": "pt"})
        if os.path.isfile(index):
            os.remove(index)
        return single
    size = {k: v.numel() * v.element_size() for k, v in tensors.items()}
    total = sum(size.values())
    parts: list[dict[str, torch.Tensor]] = [{} for _ in range(shards)]
    done = 0
    for name in sorted(tensors):
        parts[min(shards - 1, done * shards // max(1, total))][name] = tensors[name].contiguous()
        done += size[name]
    parts = [p for p in parts if p]
    weight_map = {}
    for i, part in enumerate(parts):
        fname = f"model-{i + 1:05d}-of-{len(parts):05d}.safetensors"
        save_file(part, os.path.join(folder, fname), metadata={"format": "pt"})
        weight_map.update({name: fname for name in part})
    with open(index, "w") as f:
        json.dump({"metadata": {"total_size": total}, "weight_map": weight_map}, f, indent=1)
    if os.path.isfile(single):
        os.remove(single)
    return index

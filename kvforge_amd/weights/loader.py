"""Loads a model's tensors by name and checks them against what its parts expect.

Run-time dtypes: under a bfloat16 engine, 16-bit floating tensors are kept in bfloat16 and a
tensor the checkpoint stores in 32-bit stays 32-bit; under a float32 engine every floating
tensor is widened to float32 (exact).  Integer tensors become int32 tables.  Missing tensors,
unexpected tensors and wrong shapes are reported together in one ``WeightsError``; the
reference only reports missing keys (src/tokenvault/model_loader.py:107-111).
"""

from __future__ import annotations

import re

import torch

from kvforge_amd.parts.base import ModelSpec, WeightSpec
from kvforge_amd.weights.io import WeightsError, read_tensors, tensor_index

_FLOAT_STORED = {"F32", "F16", "BF16", "F64"}
_INT_STORED = {"I64", "I32", "I16", "I8", "U8"}


def check_index(expected: dict[str, WeightSpec], index: dict[str, tuple], ignored: tuple[str, ...]
                ) -> None:
    missing = sorted(n for n in expected if n not in index)
    pats = [re.compile(p) for p in ignored]
    unexpected = sorted(n for n in index if n not in expected and not any(p.fullmatch(n) for p in pats))
    wrong: list[str] = []
    for name, spec in expected.items():
        if name not in index:
            continue
        _, shape, dt = index[name]
        if tuple(shape) != tuple(spec.shape):
            wrong.append(f"{name}: expected {list(spec.shape)}, found {list(shape)}")
        elif spec.integer and dt not in _INT_STORED:
            wrong.append(f"{name}: expected an integer table, found {dt}")
        elif not spec.integer and dt not in _FLOAT_STORED:
            wrong.append(f"{name}: expected a floating tensor, found {dt}")
    if missing or unexpected or wrong:
        lines = ["checkpoint does not match the model:"]
        if missing:
            lines.append(f"  missing tensors ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            lines.append(f"  unexpected tensors ({len(unexpected)}): " + ", ".join(unexpected))
        if wrong:
            lines.append(f"  wrong shapes or types ({len(wrong)}): " + "; ".join(wrong))
        raise WeightsError("\n".join(lines))


def runtime_dtype(stored: torch.dtype, engine_dtype: torch.dtype) -> torch.dtype:
    if not stored.is_floating_point:
        return torch.int32
    if engine_dtype == torch.float32:
        return torch.float32
    return torch.float32 if stored in (torch.float32, torch.float64) else torch.bfloat16


def load_model_weights(spec: ModelSpec, folder: str, engine_dtype: torch.dtype,
                       device: torch.device | str) -> None:
    """Read, check, convert, move to the device and hand every part its tensors."""
    expected = spec.weight_specs()
    check_index(expected, tensor_index(folder), spec.ignored_weights)
    raw = read_tensors(folder, list(expected))
    tensors = {name: t.to(device=device, dtype=runtime_dtype(t.dtype, engine_dtype)).contiguous()
               for name, t in raw.items()}
    del raw
    for part in spec.all_parts():
        part.load(tensors)

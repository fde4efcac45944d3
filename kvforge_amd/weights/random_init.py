"""Random-weights mode: writes a model folder (``config.json``, ``model.safetensors``) from a
configuration and a seed.

The reference's ``build_model`` (src/tokenvault/model_loader.py:42-61) draws every matrix from
N(0, 0.02) under one seed and sets norm weights to a constant.  Here norm weights are drawn from
1 + N(0, 0.1), because a kernel that forgets a constant-one weight still passes, and the tensors
go through the same files and loader as a real checkpoint.
"""

from __future__ import annotations

from typing import Any

import torch

from kvforge_amd import registry
from kvforge_amd.weights.io import write_safetensors

_STORE = {"bfloat16": torch.bfloat16, "float32": torch.float32,
          torch.bfloat16: torch.bfloat16, torch.float32: torch.float32}


def _stored_as(dtype: "str | torch.dtype") -> torch.dtype:
    try:
        return _STORE[dtype]
    except KeyError:
        raise ValueError(f"random weights are stored as bfloat16 or float32, not {dtype!r}") from None


def random_tensors(spec, seed: int, dtype: "str | torch.dtype" = "bfloat16") -> dict[str, torch.Tensor]:
    """Tensors for every name the model expects, drawn in 32-bit in sorted name order from one
    generator and stored as ``dtype`` (the reference draws in 32-bit and casts to the engine's
    type, src/tokenvault/model_loader.py:55-61)."""
    store = _stored_as(dtype)
    gen = torch.Generator().manual_seed(int(seed))
    out: dict[str, torch.Tensor] = {}
    for name, w in sorted(spec.weight_specs().items()):
        if w.integer:
            out[name] = torch.zeros(w.shape, dtype=torch.int32)
        elif w.init == "zeros":
            out[name] = torch.zeros(w.shape, dtype=store)
        else:
            t = torch.randn(w.shape, generator=gen, dtype=torch.float32) * w.std
            if w.init == "norm":
                t = t + 1.0
            elif w.init != "normal":
                raise ValueError(f"unknown init {w.init!r} for {name}")
            out[name] = t.to(store)
    return out


def write_random_model(folder: str, config: "dict[str, Any] | Any", seed: int = 0,
                       dtype: "str | torch.dtype" = "bfloat16") -> str:
    """``config``: a config.json dictionary or a typed configuration.  ``dtype``: what the
    file stores; a float32 engine should be given ``"float32"``, or it only ever meets numbers
    that bfloat16 can hold (``InferenceEngine.from_config`` passes its own type)."""
    cfg = registry.config_from_dict(config) if isinstance(config, dict) else config
    spec = registry.build_spec(cfg)
    cfg.save(folder)
    write_safetensors(folder, random_tensors(spec, seed, dtype))
    return folder


def load_random_weights(spec, seed: int, engine_dtype: torch.dtype, device: "torch.device | str",
                        dtype: "str | torch.dtype | None" = None) -> dict[str, torch.Tensor]:
    """The random-weights mode without the files, for models too large to be worth writing:
    every tensor of ``spec`` is drawn on ``device`` (same laws, same name order, stored in
    ``dtype``, by default the engine's own, and then held as the loader would hold a tensor
    stored so) and handed to the parts.  The device's generator gives other numbers than
    ``write_random_model`` does for the same seed.  Returns the tensors by checkpoint name, as
    drawn (the parts keep layouts of their own)."""
    from kvforge_amd.weights.loader import runtime_dtype

    store = _stored_as(engine_dtype if dtype is None else dtype)
    gen = torch.Generator(device=device).manual_seed(int(seed))
    tensors: dict[str, torch.Tensor] = {}
    for name, w in sorted(spec.weight_specs().items()):
        if w.integer:
            tensors[name] = torch.zeros(w.shape, dtype=torch.int32, device=device)
            continue
        if w.init == "zeros":
            t = torch.zeros(w.shape, dtype=torch.float32, device=device)
        elif w.init in ("normal", "norm"):
            t = torch.randn(w.shape, generator=gen, dtype=torch.float32, device=device) * w.std
            if w.init == "norm":
                t += 1.0
        else:
            raise ValueError(f"unknown init {w.init!r} for {name}")
        tensors[name] = t.to(store).to(runtime_dtype(store, engine_dtype)).contiguous()
    for part in spec.all_parts():
        part.load(tensors)
    return tensors

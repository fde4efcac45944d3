"""Typed model configuration read from an architecture's own ``config.json`` keys.

Behaviour follows the reference's ``ModelConfig`` (src/tokenvault/config.py:34-72) and its
HF-key mapping (src/tokenvault/model_loader.py:64-86): ``head_dim`` defaults to
``hidden_size / num_attention_heads``, ``num_key_value_heads`` defaults to the number of
heads, query heads must be a multiple of key/value heads.  The reference never reads
``rope_scaling``; the llama3 rule is added here because the Llama 3.x checkpoints need it.

No size lives in code: every number a part needs comes from these dataclasses, which are
filled from ``config.json`` (or from a preset that is itself written as ``config.json``).
"""

from __future__ import annotations

import json
import os
from dataclasses import dataclass, field
from typing import Any, ClassVar


class ConfigError(ValueError):
    """A ``config.json`` that cannot describe a model this framework can run."""


@dataclass(frozen=True)
class RopeScaling:
    """Frequency rescaling of rotary embeddings (``rope_scaling`` in config.json).

    ``rope_type`` ``"llama3"``: wavelengths longer than ``original_max_position_embeddings /
    low_freq_factor`` are divided by ``factor``; wavelengths shorter than
    ``original_max_position_embeddings / high_freq_factor`` are kept; in between the two are
    blended linearly in ``original_max_position_embeddings / wavelength``.
    """

    rope_type: str
    factor: float
    low_freq_factor: float = 1.0
    high_freq_factor: float = 4.0
    original_max_position_embeddings: int = 8192

    KNOWN: ClassVar[tuple[str, ...]] = ("llama3",)

    @classmethod
    def from_dict(cls, d: dict[str, Any] | None) -> "RopeScaling | None":
        if d is None:
            return None
        kind = d.get("rope_type", d.get("type"))
        if kind in (None, "default"):
            return None
        if kind not in cls.KNOWN:
            raise ConfigError(f"rope_scaling type {kind!r} is not supported (known: {cls.KNOWN})")
        try:
            return cls(
                rope_type=kind,
                factor=float(d["factor"]),
                low_freq_factor=float(d["low_freq_factor"]),
                high_freq_factor=float(d["high_freq_factor"]),
                original_max_position_embeddings=int(d["original_max_position_embeddings"]),
            )
        except KeyError as e:
            raise ConfigError(f"rope_scaling of type {kind!r} needs key {e.args[0]!r}") from None

    def to_dict(self) -> dict[str, Any]:
        return {
            "rope_type": self.rope_type,
            "factor": self.factor,
            "low_freq_factor": self.low_freq_factor,
            "high_freq_factor": self.high_freq_factor,
            "original_max_position_embeddings": self.original_max_position_embeddings,
        }


@dataclass
class ModelConfig:
    """What every architecture's configuration has: a registry key and a vocabulary.

    Sub-classes add their own typed fields and implement :meth:`from_dict` / :meth:`to_dict`
    in terms of the key names their ``config.json`` uses.
    """

    architecture: str
    vocab_size: int
    max_position_embeddings: int
    bos_token_id: int | None = None
    eos_token_id: int | None = None

    @classmethod
    def from_dict(cls, d: dict[str, Any]) -> "ModelConfig":  # pragma: no cover - abstract
        raise NotImplementedError

    def to_dict(self) -> dict[str, Any]:  # pragma: no cover - abstract
        raise NotImplementedError

    def save(self, folder: str) -> str:
        os.makedirs(folder, exist_ok=True)
        path = os.path.join(folder, "config.json")
        with open(path, "w") as f:
            json.dump(self.to_dict(), f, indent=2)
        return path


def _require(d: dict[str, Any], key: str) -> Any:
    if key not in d or d[key] is None:
        raise ConfigError(f"config.json lacks the key {key!r}")
    return d[key]


def _first(x: Any) -> Any:
    # eos_token_id may be a list in config.json; the reference takes its first element
    # (src/tokenvault/model_loader.py:68).
    return x[0] if isinstance(x, (list, tuple)) and x else x


@dataclass
class LlamaConfig(ModelConfig):
    """Dense Llama decoder: pre-norm RMSNorm, rotary positions, grouped-query attention,
    SwiGLU feed-forward (the model of src/tokenvault/model.py:146-191).

    ``sliding_window`` / ``layer_types`` are optional keys: a layer whose type is
    ``"sliding_attention"`` attends to the last ``sliding_window`` keys only.  Llama
    checkpoints do not carry them; they exist so that one model can hold two kinds of
    attention layer with cache groups of their own.
    """

    hidden_size: int = 0
    num_hidden_layers: int = 0
    num_attention_heads: int = 0
    num_key_value_heads: int = 0
    head_dim: int = 0
    intermediate_size: int = 0
    rms_norm_eps: float = 0.0
    rope_theta: float = 10000.0
    rope_scaling: RopeScaling | None = None
    hidden_act: str = "silu"
    tie_word_embeddings: bool = False
    sliding_window: int | None = None
    layer_types: list[str] | None = None
    torch_dtype: str | None = None

    def __post_init__(self) -> None:
        H, KV = self.num_attention_heads, self.num_key_value_heads
        for name in ("vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads",
                     "num_key_value_heads", "head_dim", "intermediate_size",
                     "max_position_embeddings"):
            if int(getattr(self, name)) <= 0:
                raise ConfigError(f"{name} must be positive, got {getattr(self, name)}")
        if H % KV != 0:
            raise ConfigError(
                f"num_attention_heads ({H}) must be a multiple of num_key_value_heads ({KV})")
        if self.head_dim % 2 != 0:
            raise ConfigError(f"head_dim ({self.head_dim}) must be even for rotary embeddings")
        if not self.rms_norm_eps > 0:
            raise ConfigError("rms_norm_eps must be positive")
        if self.hidden_act != "silu":
            raise ConfigError(f"hidden_act {self.hidden_act!r} is not supported (known: 'silu')")
        if self.layer_types is not None:
            if len(self.layer_types) != self.num_hidden_layers:
                raise ConfigError("layer_types must name every layer")
            for t in self.layer_types:
                if t not in ("full_attention", "sliding_attention"):
                    raise ConfigError(f"unknown layer type {t!r}")
            if "sliding_attention" in self.layer_types and not self.sliding_window:
                raise ConfigError("sliding_attention layers need sliding_window")

    @classmethod
    def from_dict(cls, d: dict[str, Any]) -> "LlamaConfig":
        archs = d.get("architectures") or ["LlamaForCausalLM"]
        hidden = int(_require(d, "hidden_size"))
        heads = int(_require(d, "num_attention_heads"))
        head_dim = d.get("head_dim")
        if head_dim is None:
            if hidden % heads != 0:
                raise ConfigError(
                    "hidden_size must be divisible by num_attention_heads when head_dim is unset")
            head_dim = hidden // heads
        for bias_key in ("attention_bias", "mlp_bias"):
            if d.get(bias_key):
                raise ConfigError(f"{bias_key}=true is not supported: projections carry no bias")
        return cls(
            architecture=archs[0],
            vocab_size=int(_require(d, "vocab_size")),
            max_position_embeddings=int(_require(d, "max_position_embeddings")),
            bos_token_id=_first(d.get("bos_token_id")),
            eos_token_id=_first(d.get("eos_token_id")),
            hidden_size=hidden,
            num_hidden_layers=int(_require(d, "num_hidden_layers")),
            num_attention_heads=heads,
            num_key_value_heads=int(d.get("num_key_value_heads") or heads),
            head_dim=int(head_dim),
            intermediate_size=int(_require(d, "intermediate_size")),
            rms_norm_eps=float(_require(d, "rms_norm_eps")),
            rope_theta=float(d.get("rope_theta", 10000.0)),
            rope_scaling=RopeScaling.from_dict(d.get("rope_scaling")),
            hidden_act=d.get("hidden_activation") or d.get("hidden_act", "silu"),
            tie_word_embeddings=bool(d.get("tie_word_embeddings", False)),
            sliding_window=d.get("sliding_window"),
            layer_types=d.get("layer_types"),
            torch_dtype=d.get("torch_dtype"),
        )

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {
            "architectures": [self.architecture],
            "model_type": "llama",
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "intermediate_size": self.intermediate_size,
            "max_position_embeddings": self.max_position_embeddings,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "rope_scaling": self.rope_scaling.to_dict() if self.rope_scaling else None,
            "hidden_act": self.hidden_act,
            "tie_word_embeddings": self.tie_word_embeddings,
            "attention_bias": False,
            "mlp_bias": False,
            "bos_token_id": self.bos_token_id,
            "eos_token_id": self.eos_token_id,
        }
        if self.sliding_window is not None:
            out["sliding_window"] = self.sliding_window
        if self.layer_types is not None:
            out["layer_types"] = list(self.layer_types)
        if self.torch_dtype is not None:
            out["torch_dtype"] = self.torch_dtype
        return out

    @property
    def num_params(self) -> int:
        """Parameter count without norms (src/tokenvault/config.py:64-72)."""
        h, d = self.hidden_size, self.head_dim
        attn = h * d * (self.num_attention_heads * 2 + self.num_key_value_heads * 2)
        mlp = 3 * h * self.intermediate_size
        emb = self.vocab_size * h * (1 if self.tie_word_embeddings else 2)
        return self.num_hidden_layers * (attn + mlp) + emb


def read_config_json(folder_or_file: str) -> dict[str, Any]:
    path = folder_or_file
    if os.path.isdir(path):
        path = os.path.join(path, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"no config.json at {path}")
    with open(path) as f:
        d = json.load(f)
    if not isinstance(d, dict):
        raise ConfigError(f"{path} does not hold a JSON object")
    return d

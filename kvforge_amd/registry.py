"""One registry from an architecture's name (``architectures[0]`` of config.json) to its typed
configuration and the builder that assembles its model from parts; and registries of the parts
themselves by kind, so a builder can choose a mixer, feed-forward, norm or position encoding
layer by layer from what the configuration says.

The reference has no registry: one hard-wired ``Transformer`` serves every checkpoint and
sniffs ``model_type`` (src/tokenvault/model_loader.py:65-66).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable

from kvforge_amd.config.model import ConfigError, ModelConfig, read_config_json


@dataclass(frozen=True)
class Architecture:
    name: str
    config_cls: type
    build: Callable[[Any], Any]  # typed config -> parts.base.ModelSpec


ARCHITECTURES: dict[str, Architecture] = {}
MIXERS: dict[str, type] = {}
FEED_FORWARDS: dict[str, type] = {}
NORMS: dict[str, type] = {}
POSITIONS: dict[str, type] = {}
BLOCKS: dict[str, type] = {}


def register_architecture(name: str, config_cls: type, build: Callable[[Any], Any]) -> None:
    ARCHITECTURES[name] = Architecture(name, config_cls, build)


def _registrar(table: dict[str, type]):
    def register(kind: str, cls: type | None = None):
        if cls is not None:
            table[kind] = cls
            return cls

        def deco(c: type) -> type:
            table[kind] = c
            return c
        return deco
    return register


register_mixer = _registrar(MIXERS)
register_feed_forward = _registrar(FEED_FORWARDS)
register_norm = _registrar(NORMS)
register_positions = _registrar(POSITIONS)
register_block = _registrar(BLOCKS)


def part_class(table: dict[str, type], kind: str, what: str) -> type:
    try:
        return table[kind]
    except KeyError:
        raise ConfigError(f"unknown {what} {kind!r}; registered: {sorted(table)}") from None


def get_architecture(name: str) -> Architecture:
    _ensure_builtin()
    try:
        return ARCHITECTURES[name]
    except KeyError:
        raise ConfigError(
            f"architecture {name!r} is not registered; known: {sorted(ARCHITECTURES)}") from None


def config_from_dict(d: dict[str, Any]) -> ModelConfig:
    archs = d.get("architectures")
    if not archs:
        raise ConfigError("config.json lacks 'architectures'")
    return get_architecture(archs[0]).config_cls.from_dict(d)


def config_from_folder(folder: str) -> ModelConfig:
    return config_from_dict(read_config_json(folder))


def build_spec(config: ModelConfig):
    return get_architecture(config.architecture).build(config)


_builtin_done = False


def _ensure_builtin() -> None:
    global _builtin_done
    if not _builtin_done:
        _builtin_done = True
        import kvforge_amd.parts  # noqa: F401  registers the parts
        import kvforge_amd.models  # noqa: F401  registers the architectures

"""kvforge_amd: a small, whole LLM inference engine for one MI355X (gfx950).

A model folder (config.json + safetensors) goes in, tokens come out: typed configuration and an
architecture registry, weights by tensor name, parts assembled into a transformer, a paged cache
with block tables, one step function over flat mixed batches, a token-budget scheduler, sampling,
and hand-written HIP kernels for everything between a request's tokens and its next token.
"""

from kvforge_amd.config import (PRESETS, CacheConfig, ConfigError, EngineConfig, LlamaConfig,
                                ModelConfig, RopeScaling, SchedulerConfig, SchedulingPolicy,
                                preset_dict)
from kvforge_amd.registry import (config_from_dict, config_from_folder, get_architecture,
                                  register_architecture, register_block, register_feed_forward,
                                  register_mixer, register_norm, register_positions)
from kvforge_amd.weights import WeightsError, read_safetensors_folder, write_random_model

__version__ = "0.1.0"

_LAZY = {
    "InferenceEngine": "kvforge_amd.engine.engine",
    "SamplingParams": "kvforge_amd.sampling.params",
    "Request": "kvforge_amd.engine.request",
    "RequestOutput": "kvforge_amd.engine.request",
    "RequestStatus": "kvforge_amd.engine.request",
    "FinishReason": "kvforge_amd.engine.request",
    "Scheduler": "kvforge_amd.engine.scheduler",
    "RequestRejectedError": "kvforge_amd.engine.scheduler",
    "ModelRunner": "kvforge_amd.engine.runner",
    "StepEntry": "kvforge_amd.engine.batch",
    "Transformer": "kvforge_amd.models.transformer",
    "ByteTokenizer": "kvforge_amd.tokenizer",
    "FileTokenizer": "kvforge_amd.tokenizer",
}


def __getattr__(name):
    if name in _LAZY:
        import importlib

        return getattr(importlib.import_module(_LAZY[name]), name)
    raise AttributeError(f"module 'kvforge_amd' has no attribute {name!r}")


__all__ = ["PRESETS", "CacheConfig", "ConfigError", "EngineConfig", "LlamaConfig", "ModelConfig",
           "RopeScaling", "SchedulerConfig", "SchedulingPolicy", "preset_dict",
           "config_from_dict", "config_from_folder", "get_architecture", "register_architecture",
           "register_block", "register_feed_forward", "register_mixer", "register_norm",
           "register_positions", "WeightsError", "read_safetensors_folder", "write_random_model",
           "__version__", *sorted(_LAZY)]

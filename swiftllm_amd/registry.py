"""Model registry: which configuration class and which worker class serve a checkpoint directory.

The key is config.json's `architecture` (when present) or HuggingFace's `model_type`. The engine, the examples and the
command-line tools build their model through `build_model(engine_config)`; adding a design means adding a row here, its
configuration class in model_config.py and its worker class under worker/.
"""
import importlib
import json
import os

# key -> (configuration class, worker class), both as "module:attribute" (workers import torch and the HIP library lazily)
MODELS = {
    "llama": ("swiftllm_amd.model_config:LlamaModelConfig", "swiftllm_amd.worker.model:LlamaModel"),
    "Kekapel": ("swiftllm_amd.model_config:KekapelModelConfig", "swiftllm_amd.worker.kekapel_model:KekapelModel"),
    "Lorulix": ("swiftllm_amd.model_config:LorulixModelConfig", "swiftllm_amd.worker.lorulix_model:LorulixModel"),
    "Rosilix": ("swiftllm_amd.model_config:RosilixModelConfig", "swiftllm_amd.worker.rosilix_model:RosilixModel"),
    "Ratilorn": ("swiftllm_amd.model_config:RatilornModelConfig", "swiftllm_amd.worker.ratilorn_model:RatilornModel"),
}


def _resolve(spec: str):
    module, attr = spec.split(":")
    return getattr(importlib.import_module(module), attr)


def read_config(model_path: str) -> dict:
    with open(os.path.join(model_path, "config.json"), "r", encoding="utf-8") as f:
        return json.load(f)


def architecture_of(config: dict) -> str:
    key = config.get("architecture") or config.get("model_type")
    if key not in MODELS:
        raise ValueError(f"no model registered for architecture {key!r} (known: {sorted(MODELS)})")
    return key


def load_model_config(model_path: str):
    config = read_config(model_path)
    return _resolve(MODELS[architecture_of(config)][0])(config)


def model_class(model_path: str):
    return _resolve(MODELS[architecture_of(read_config(model_path))][1])


def build_model(engine_config):
    """The worker object for engine_config.model_path (weights not loaded yet)."""
    return model_class(engine_config.model_path)(engine_config)

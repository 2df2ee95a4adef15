"""Model registry: architecture name -> config reader and model class.

``config.json`` of a model folder names its family in "architecture"; the
reader registered for that family turns the file into a `ModelConfig`, and
`build_model` instantiates the class registered for `cfg.architecture`.
Llama-style presets have no folder and go straight to `build_model`.
"""

from __future__ import annotations

import json
import os
from typing import Callable, Dict, Tuple

from .config import ModelConfig

# name -> (config reader or None, model factory)
_REGISTRY: Dict[str, Tuple[Callable, Callable]] = {}


def register_architecture(name: str, read_config, factory) -> None:
    _REGISTRY[name.lower()] = (read_config, factory)


def _llama_factory(cfg, device, dtype, tp):
    if cfg.is_moe:
        from .mixtral import MixtralForCausalLM

        return MixtralForCausalLM(cfg, device=device, dtype=dtype, tp=tp)
    from .llama import LlamaForCausalLM

    return LlamaForCausalLM(cfg, device=device, dtype=dtype, tp=tp)


def _tikarax_factory(cfg, device, dtype, tp):
    from .tikarax import TikaraxForCausalLM

    return TikaraxForCausalLM(cfg, device=device, dtype=dtype, tp=tp)


def _tikarax_config(raw: dict, path: str) -> ModelConfig:
    from .tikarax import config_from_json

    return config_from_json(raw, path)


def _lopovik_factory(cfg, device, dtype, tp):
    from .lopovik import LopovikForCausalLM

    return LopovikForCausalLM(cfg, device=device, dtype=dtype, tp=tp)


def _lopovik_config(raw: dict, path: str) -> ModelConfig:
    from .lopovik import config_from_json

    return config_from_json(raw, path)


def _potatar_factory(cfg, device, dtype, tp):
    from .potatar import PotatarForCausalLM

    return PotatarForCausalLM(cfg, device=device, dtype=dtype, tp=tp)


def _potatar_config(raw: dict, path: str) -> ModelConfig:
    from .potatar import config_from_json

    return config_from_json(raw, path)


def _vemenex_factory(cfg, device, dtype, tp):
    from .vemenex import VemenexForCausalLM

    return VemenexForCausalLM(cfg, device=device, dtype=dtype, tp=tp)


def _vemenex_config(raw: dict, path: str) -> ModelConfig:
    from .vemenex import config_from_json

    return config_from_json(raw, path)


register_architecture("llama", None, _llama_factory)
register_architecture("vemenex", _vemenex_config, _vemenex_factory)
register_architecture("potatar", _potatar_config, _potatar_factory)
register_architecture("lopovik", _lopovik_config, _lopovik_factory)
register_architecture("tikarax", _tikarax_config, _tikarax_factory)


def config_from_dir(path: str) -> ModelConfig:
    with open(os.path.join(path, "config.json")) as f:
        raw = json.load(f)
    arch = str(raw.get("architecture", "")).lower()
    if arch not in _REGISTRY or _REGISTRY[arch][0] is None:
        raise KeyError(
            f"config.json names architecture {raw.get('architecture')!r}; "
            f"readers exist for {sorted(k for k, v in _REGISTRY.items() if v[0])}"
        )
    return _REGISTRY[arch][0](raw, path)


def build_model(cfg: ModelConfig, device, dtype, tp=None):
    arch = cfg.architecture.lower()
    if arch not in _REGISTRY:
        raise KeyError(f"unknown architecture {cfg.architecture!r}")
    model = _REGISTRY[arch][1](cfg, device, dtype, tp)
    if cfg.weights_path and hasattr(model, "load_weights"):
        from .loader import read_safetensors

        model.load_weights(
            read_safetensors(os.path.join(cfg.weights_path, "model.safetensors"))
        )
    return model

"""Model skeletons, caches and the registry that picks them by a checkpoint's config.json.

`MODEL_REGISTRY` maps the architecture name a config.json carries (`architectures[0]`, or `architecture`) to what serving that
family needs: how to read the config, the skeleton class, the optimize-rule file that injects the HIP operators, and the cache /
state manager.  `load_model(dir)` does what the reference's local_chat.py does by hand for its families: config -> skeleton on the
meta device -> rules -> weights (archive/ktransformers/local_chat.py:60-110, its `custom_models` table)."""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Callable

import torch

RULES_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "optimize", "optimize_rules")


@dataclass
class ModelEntry:
    make_config: Callable      # (config dict, compute dtype) -> config namespace
    model_class: Callable      # () -> class (imported lazily)
    rule_file: str
    make_cache: Callable       # (config, max_tokens, max_requests, dtype, device) -> cache / state manager
    dtypes: tuple = (torch.bfloat16,)


def _deepseek_config(d, dtype):
    from ktransformers_amd.models.modeling_deepseek import make_config
    return make_config(**{k: v for k, v in d.items() if k != "torch_dtype"})


def _deepseek_cache(config, max_tokens, max_requests, dtype, device):
    from ktransformers_amd.models.custom_cache import StaticCache
    return StaticCache(config, 1, max_tokens, device, dtype)


def _mixtral_config(d, dtype):
    from ktransformers_amd.models.modeling_mixtral import make_mixtral_config
    return make_mixtral_config(**{k: v for k, v in d.items() if k != "torch_dtype"})


def _mixtral_cache(config, max_tokens, max_requests, dtype, device):
    from ktransformers_amd.models.modeling_mixtral import MixtralKVCache
    return MixtralKVCache(config, max_tokens, device, dtype)


def _mitotar_config(d, dtype):
    from ktransformers_amd.models.modeling_mitotar import make_mitotar_config
    return make_mitotar_config(d, dtype)


def _mitotar_cache(config, max_tokens, max_requests, dtype, device):
    from ktransformers_amd.models.custom_cache import KHybridCache
    from ktransformers_amd.models.modeling_mitotar import mitotar_layer_specs
    return KHybridCache(mitotar_layer_specs(config), max_tokens, max_requests=max_requests, dtype=dtype, device=device)


def _pilavik_config(d, dtype):
    from ktransformers_amd.models.modeling_pilavik import make_pilavik_config
    return make_pilavik_config(d, dtype)


def _pilavik_cache(config, max_tokens, max_requests, dtype, device):
    from ktransformers_amd.models.custom_cache import KHybridCache
    from ktransformers_amd.models.modeling_pilavik import pilavik_layer_specs
    return KHybridCache(pilavik_layer_specs(config), max_tokens, max_requests=max_requests, dtype=dtype, device=device)


def _sadosun_config(d, dtype):
    from ktransformers_amd.models.modeling_sadosun import make_sadosun_config
    return make_sadosun_config(d, dtype)


def _sadosun_cache(config, max_tokens, max_requests, dtype, device):
    from ktransformers_amd.models.custom_cache import KHybridCache
    from ktransformers_amd.models.modeling_sadosun import sadosun_layer_specs
    return KHybridCache(sadosun_layer_specs(config), max_tokens, max_requests=max_requests, dtype=dtype, device=device)


def _vigodra_config(d, dtype):
    from ktransformers_amd.models.modeling_vigodra import make_vigodra_config
    return make_vigodra_config(d, dtype)


def _vigodra_cache(config, max_tokens, max_requests, dtype, device):
    from ktransformers_amd.models.custom_cache import KHybridCache
    from ktransformers_amd.models.modeling_vigodra import vigodra_layer_specs
    return KHybridCache(vigodra_layer_specs(config), max_tokens, max_requests=max_requests, dtype=dtype, device=device)


def _cls(module: str, name: str):
    def get():
        import importlib
        return getattr(importlib.import_module(module), name)
    return get


_DS = ModelEntry(_deepseek_config, _cls("ktransformers_amd.models.modeling_deepseek", "DeepseekForCausalLM"), "DeepSeek-V3-Chat.yaml",
                 _deepseek_cache)
MODEL_REGISTRY = {
    "DeepseekV3ForCausalLM": _DS,
    "DeepseekV2ForCausalLM": ModelEntry(_deepseek_config, _DS.model_class, "DeepSeek-V2-Lite-Chat.yaml", _deepseek_cache),
    "MixtralForCausalLM": ModelEntry(_mixtral_config, _cls("ktransformers_amd.models.modeling_mixtral", "MixtralForCausalLM"),
                                     "Mixtral-8x7B.yaml", _mixtral_cache),
    "Mitotar": ModelEntry(_mitotar_config, _cls("ktransformers_amd.models.modeling_mitotar", "MitotarForCausalLM"), "Mitotar.yaml",
                          _mitotar_cache, dtypes=(torch.bfloat16, torch.float32)),
    "Pilavik": ModelEntry(_pilavik_config, _cls("ktransformers_amd.models.modeling_pilavik", "PilavikForCausalLM"), "Pilavik.yaml",
                          _pilavik_cache, dtypes=(torch.bfloat16, torch.float32)),
    "Sadosun": ModelEntry(_sadosun_config, _cls("ktransformers_amd.models.modeling_sadosun", "SadosunForCausalLM"), "Sadosun.yaml",
                          _sadosun_cache, dtypes=(torch.bfloat16, torch.float32)),
    "Vigodra": ModelEntry(_vigodra_config, _cls("ktransformers_amd.models.modeling_vigodra", "VigodraForCausalLM"), "Vigodra.yaml",
                          _vigodra_cache, dtypes=(torch.bfloat16, torch.float32)),
}


def architecture_of(config: dict) -> str:
    arch = config.get("architecture") or (config.get("architectures") or [None])[0]
    if arch not in MODEL_REGISTRY:
        raise KeyError(f"no model registered for architecture {arch!r} (known: {sorted(MODEL_REGISTRY)})")
    return arch


def read_config(model_dir: str) -> dict:
    with open(os.path.join(model_dir, "config.json"), encoding="utf-8") as f:
        return json.load(f)


def load_model(model_dir: str, dtype=torch.bfloat16, device: str = "cuda:0", rule_file: str | None = None, loader=None):
    """(model with its operators injected and weights loaded, config, registry entry) for the checkpoint folder `model_dir`
    (config.json + *.safetensors).  `loader`: a weight source with the loader protocol (util/loader.py) instead of the folder's
    safetensors files."""
    from ktransformers_amd.optimize.optimize import optimize_and_load
    from ktransformers_amd.util.loader import SafeTensorLoader

    raw = read_config(model_dir) if isinstance(model_dir, str) else model_dir
    entry = MODEL_REGISTRY[architecture_of(raw)]
    if dtype not in entry.dtypes:
        raise ValueError(f"{architecture_of(raw)} runs in {entry.dtypes}, not {dtype}")
    config = entry.make_config(raw, dtype)
    with torch.device("meta"):
        model = entry.model_class()(config)
    if loader is None:
        loader = SafeTensorLoader(model_dir)
    rules = rule_file or os.path.join(RULES_DIR, entry.rule_file)
    optimize_and_load(model, rules, loader, config, default_device=device)
    return model, config, entry

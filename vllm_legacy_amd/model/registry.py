"""Model registry: config.json's architecture name -> how to build the model, read its
configuration and fill it from a checkpoint folder.  The engine looks models up here and
nowhere else (the role of the reference's ModelRegistry, vllm/model_executor/models/__init__.py)."""
import importlib
import json
import os
from typing import Callable, Dict, Tuple

import torch

# architecture -> (module, model class, config class)
_MODELS: Dict[str, Tuple[str, str, str]] = {
    "Lusadra": ("vllm_legacy_amd.model.lusadra", "LusadraForCausalLM", "LusadraConfig"),
    "Dopipel": ("vllm_legacy_amd.model.dopipel", "DopipelForCausalLM", "DopipelConfig"),
    "Lamosun": ("vllm_legacy_amd.model.lamosun", "LamosunForCausalLM", "LamosunConfig"),
    "Tekezen": ("vllm_legacy_amd.model.tekezen", "TekezenForCausalLM", "TekezenConfig"),
    # the synthetic-weight Llama stack behind the engine's model protocol
    "LlamaDecodeStack": ("vllm_legacy_amd.engine.llama_adapter", "PagedLlamaForEngine", "LlamaEngineConfig"),
}


def register_model(architecture: str, module: str, model_cls: str, config_cls: str) -> None:
    _MODELS[architecture] = (module, model_cls, config_cls)


def supported_architectures():
    return sorted(_MODELS)


def resolve(architecture: str):
    if architecture not in _MODELS:
        raise ValueError(f"Model architecture {architecture!r} is not supported; "
                         f"supported: {supported_architectures()}")
    module, model_cls, config_cls = _MODELS[architecture]
    mod = importlib.import_module(module)
    return getattr(mod, model_cls), getattr(mod, config_cls)


def architecture_of(config: Dict) -> str:
    if "architecture" in config:
        return config["architecture"]
    archs = config.get("architectures") or []
    if archs:
        return archs[0]
    raise ValueError("config.json names no architecture")


def load_model(model_dir: str, dtype: torch.dtype = torch.bfloat16, device="cuda"):
    """Build the model a folder's config.json names and fill it from its model.safetensors
    (a folder without one gets the model's own random weights: synthetic stacks)."""
    from vllm_legacy_amd.model_loader.safetensors_file import load_safetensors
    with open(os.path.join(model_dir, "config.json")) as f:
        raw = json.load(f)
    model_cls, config_cls = resolve(architecture_of(raw))
    cfg = config_cls.from_dict(raw)
    model = model_cls(cfg, dtype=dtype, device=device)
    weights = os.path.join(model_dir, "model.safetensors")
    if os.path.exists(weights):
        model.load_weights(load_safetensors(weights))
    return model

"""Model registry: config.json's architecture name -> the loader that turns a checkpoint directory into the engine's
(language model, vision model or None) pair.  The reference picks its model class the same way, from the HF config's
`architectures` (hydrainfer/model/model_factory.py); here a design is added with `register`."""
import json
import os
from typing import Callable, Dict, Optional, Tuple

import torch

_LOADERS: Dict[str, Callable] = {}


def register(architecture: str, loader: Callable) -> None:
    """loader(model_path, dtype, device, **options) -> (language model for the engine, vision model or None)."""
    _LOADERS[architecture] = loader


def architecture_of(model_path: str) -> str:
    with open(os.path.join(model_path, "config.json")) as f:
        cfg = json.load(f)
    name = cfg.get("architecture") or (cfg.get("architectures") or [None])[0]
    if name is None and ("text_config" in cfg or "vision_config" in cfg):
        name = "LlavaForConditionalGeneration"      # a LLaVA configuration written without its class name
    if name is None:
        raise ValueError(f"{model_path}/config.json names no architecture")
    return name


def registered() -> Tuple[str, ...]:
    return tuple(sorted(_LOADERS))


def load_model(model_path: str, dtype: torch.dtype, device, **options):
    name = architecture_of(model_path)
    if name not in _LOADERS:
        raise ValueError(f"unknown architecture {name!r}; registered: {', '.join(registered())}")
    return _LOADERS[name](model_path, dtype, device, **options)


def _load_llava(model_path: str, dtype, device, vision: bool = True, language: bool = True):
    from hydrainfer_amd.model.loader import load_llava
    return load_llava(model_path, dtype, device, vision=vision, language=language)


def _load_tetepel(model_path: str, dtype, device, **_):
    from hydrainfer_amd.model.llava import TextLanguageModel
    from hydrainfer_amd.model.loader import scan_safetensors
    from hydrainfer_amd.model.tetepel import TetepelForCausalLM, read_shape
    shape = read_shape(model_path)
    model = TetepelForCausalLM.from_state_dict(shape, scan_safetensors(model_path, ("",)), dtype, device)
    return TextLanguageModel(model), None


def _load_kezolix(model_path: str, dtype, device, **_):
    from hydrainfer_amd.model.kezolix import KezolixForCausalLM, read_shape
    from hydrainfer_amd.model.llava import TextLanguageModel
    from hydrainfer_amd.model.loader import scan_safetensors
    shape = read_shape(model_path)
    model = KezolixForCausalLM.from_state_dict(shape, scan_safetensors(model_path, ("",)), dtype, device)
    return TextLanguageModel(model), None


def _load_fasanex(model_path: str, dtype, device, **_):
    from hydrainfer_amd.model.fasanex import FasanexForCausalLM, read_shape
    from hydrainfer_amd.model.llava import TextLanguageModel
    from hydrainfer_amd.model.loader import scan_safetensors
    shape = read_shape(model_path)
    model = FasanexForCausalLM.from_state_dict(shape, scan_safetensors(model_path, ("",)), dtype, device)
    return TextLanguageModel(model), None


def _load_pemalorn(model_path: str, dtype, device, **_):
    from hydrainfer_amd.model.llava import TextLanguageModel
    from hydrainfer_amd.model.loader import scan_safetensors
    from hydrainfer_amd.model.pemalorn import PemalornForCausalLM, read_shape
    shape = read_shape(model_path)
    model = PemalornForCausalLM.from_state_dict(shape, scan_safetensors(model_path, ("",)), dtype, device)
    return TextLanguageModel(model), None


register("LlavaForConditionalGeneration", _load_llava)
register("Tetepel", _load_tetepel)
register("Kezolix", _load_kezolix)
register("Fasanex", _load_fasanex)
register("Pemalorn", _load_pemalorn)

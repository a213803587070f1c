"""Model registry: family name -> model class, checkpoint architecture ->
config reader.

EngineConfig.model is either a named architecture (engine.config
ARCHITECTURES) or a checkpoint folder whose config.json carries an
"architecture" (or HF "architectures") entry; the runner builds the class
registered for ModelConfig.family and loads weights through the family's
loader.
"""

from __future__ import annotations

import json
import os
from typing import Callable, Dict

import torch

from production_stack_amd.engine.config import ModelConfig


def _llama_cls():
    from production_stack_amd.engine.models.llama import LlamaForCausalLM

    return LlamaForCausalLM


def _nanurax_cls():
    from production_stack_amd.engine.models.nanurax import NanuraxForCausalLM

    return NanuraxForCausalLM


def _derusun_cls():
    from production_stack_amd.engine.models.derusun import DerusunForCausalLM

    return DerusunForCausalLM


def _bipulorn_cls():
    from production_stack_amd.engine.models.bipulorn import (
        BipulornForCausalLM,
    )

    return BipulornForCausalLM


def _dogidra_cls():
    from production_stack_amd.engine.models.dogidra import (
        DogidraForCausalLM,
    )

    return DogidraForCausalLM


MODEL_CLASSES: Dict[str, Callable] = {
    "llama": _llama_cls,
    "nanurax": _nanurax_cls,
    "derusun": _derusun_cls,
    "bipulorn": _bipulorn_cls,
    "dogidra": _dogidra_cls,
}


def _nanurax_config(path: str) -> ModelConfig:
    from production_stack_amd.engine.models import nanurax

    return nanurax.config_from_dir(path)


# config.json "architecture" -> reader(path) -> ModelConfig
def _derusun_config(path: str) -> ModelConfig:
    from production_stack_amd.engine.models import derusun

    return derusun.config_from_dir(path)


def _bipulorn_config(path: str) -> ModelConfig:
    from production_stack_amd.engine.models import bipulorn

    return bipulorn.config_from_dir(path)


def _dogidra_config(path: str) -> ModelConfig:
    from production_stack_amd.engine.models import dogidra

    return dogidra.config_from_dir(path)


CONFIG_READERS: Dict[str, Callable[[str], ModelConfig]] = {
    "Nanurax": _nanurax_config,
    "Derusun": _derusun_config,
    "Bipulorn": _bipulorn_config,
    "Dogidra": _dogidra_config,
}

# families whose layers also run in float32 (the Llama path is bf16-only)
FP32_FAMILIES = {"nanurax", "derusun", "bipulorn", "dogidra"}


def config_from_dir(path: str) -> ModelConfig:
    with open(os.path.join(path, "config.json")) as f:
        cfg = json.load(f)
    arch = cfg.get("architecture")
    if arch is None and cfg.get("architectures"):
        arch = cfg["architectures"][0]
    reader = CONFIG_READERS.get(arch)
    if reader is None:
        raise ValueError(
            f"unsupported architecture {arch!r} in {path}/config.json; "
            f"known: {sorted(CONFIG_READERS)}")
    return reader(path)


def torch_dtype(name: str) -> torch.dtype:
    try:
        return {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16,
                "float32": torch.float32, "fp32": torch.float32}[name]
    except KeyError:
        raise ValueError(f"unsupported dtype {name!r}") from None


def build_model(cfg: ModelConfig, dtype: str = "bfloat16", tp: int = 1,
                pp_rank: int = 0, pp_size: int = 1):
    if cfg.family not in MODEL_CLASSES:
        raise ValueError(f"unknown model family {cfg.family!r}")
    cls = MODEL_CLASSES[cfg.family]()
    if cfg.family in FP32_FAMILIES:
        return cls(cfg, tp=tp, pp_rank=pp_rank, pp_size=pp_size,
                   dtype=torch_dtype(dtype))
    if dtype in ("float32", "fp32"):
        raise ValueError(
            f"model family {cfg.family!r} runs in bfloat16 only")
    return cls(cfg, tp=tp, pp_rank=pp_rank, pp_size=pp_size)


def load_weights(model, path: str) -> None:
    if hasattr(model, "load_weights"):
        model.load_weights(path)
        return
    from production_stack_amd.engine.weights import load_safetensors

    load_safetensors(model, path)

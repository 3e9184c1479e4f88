"""Model registry: which model class, configuration reader and cache layout serve a checkpoint directory.

A family is chosen by config.json: `architectures[0]` (Hugging Face layout) or `architecture` (a plain string). Each entry
says how to read the configuration, how to build the model, and what the engine has to provide for it:

  * `stateful`: layers carry per-sequence state (recurrences, convolution tails) in state slots beside the paged KV cache.
    Such a model cannot take K/V of another request's identical prefix (the state is not in the pages), so the block
    manager's prefix cache is off, and every step — portions of prompts and single decoded tokens, mixed freely — goes
    through ONE packed varlen path.
  * `block_multiple`: page sizes the family's attention kernels accept (multiples of it).
  * `dtypes`: activation types the family's kernels are instantiated for.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Callable


@dataclass(frozen=True)
class ModelSpec:
    name: str
    read_config: Callable[[str, dict], object]        # (model dir, parsed config.json) -> configuration object
    build: Callable[..., object]                      # (configuration, dtype) -> nn.Module
    stateful: bool = False
    block_multiple: int = 256
    dtypes: tuple = ("bfloat16",)


def _qwen3_config(path: str, raw: dict):
    from transformers import AutoConfig
    return AutoConfig.from_pretrained(path)


def _qwen3_build(config, dtype=None):
    from .qwen3 import Qwen3ForCausalLM
    return Qwen3ForCausalLM(config)


def _foduzen_config(path: str, raw: dict):
    from .foduzen import FoduzenConfig
    return FoduzenConfig(raw)


def _foduzen_build(config, dtype=None):
    from .foduzen import FoduzenForCausalLM
    return FoduzenForCausalLM(config, dtype)


def _nokipel_config(path: str, raw: dict):
    from .nokipel import NokipelConfig
    return NokipelConfig(raw)


def _nokipel_build(config, dtype=None):
    from .nokipel import NokipelForCausalLM
    return NokipelForCausalLM(config, dtype)


def _pefazen_config(path: str, raw: dict):
    from .pefazen import PefazenConfig
    return PefazenConfig(raw)


def _pefazen_build(config, dtype=None):
    from .pefazen import PefazenForCausalLM
    return PefazenForCausalLM(config, dtype)


def _lobidra_config(path: str, raw: dict):
    from .lobidra import LobidraConfig
    return LobidraConfig(raw)


def _lobidra_build(config, dtype=None):
    from .lobidra import LobidraForCausalLM
    return LobidraForCausalLM(config, dtype)


REGISTRY: dict[str, ModelSpec] = {
    "Qwen3ForCausalLM": ModelSpec("Qwen3ForCausalLM", _qwen3_config, _qwen3_build),
    "Qwen2ForCausalLM": ModelSpec("Qwen2ForCausalLM", _qwen3_config, _qwen3_build),      # same module tree, biased qkv, no q/k norm
    "Foduzen": ModelSpec("Foduzen", _foduzen_config, _foduzen_build, stateful=True, block_multiple=16,
                         dtypes=("bfloat16", "float32")),
    "Nokipel": ModelSpec("Nokipel", _nokipel_config, _nokipel_build, stateful=True, block_multiple=16,
                         dtypes=("bfloat16", "float32")),
    "Pefazen": ModelSpec("Pefazen", _pefazen_config, _pefazen_build, stateful=True, block_multiple=16,
                         dtypes=("bfloat16", "float32")),
    "Lobidra": ModelSpec("Lobidra", _lobidra_config, _lobidra_build, stateful=True, block_multiple=16,
                         dtypes=("bfloat16", "float32")),
}


def architecture_of(raw: dict) -> str:
    if isinstance(raw.get("architecture"), str):
        return raw["architecture"]
    arch = raw.get("architectures")
    if isinstance(arch, (list, tuple)) and arch:
        return arch[0]
    raise ValueError("config.json names no architecture (`architecture` or `architectures`)")


def resolve(path: str) -> tuple[ModelSpec, object]:
    """(spec, configuration object) of the checkpoint directory `path`."""
    with open(os.path.join(path, "config.json")) as fh:
        raw = json.load(fh)
    arch = architecture_of(raw)
    if arch not in REGISTRY:
        raise ValueError(f"unsupported architecture {arch!r}; known: {sorted(REGISTRY)}")
    spec = REGISTRY[arch]
    return spec, spec.read_config(path, raw)


def spec_of(config) -> ModelSpec:
    """Spec of an already-read configuration object (Hugging Face or this package's own)."""
    arch = getattr(config, "architecture", None)
    if not isinstance(arch, str):
        archs = getattr(config, "architectures", None) or ["Qwen3ForCausalLM"]
        arch = archs[0]
    return REGISTRY.get(arch, REGISTRY["Qwen3ForCausalLM"])

"""One registry from an architecture's name to its configuration class and its model builder.

The reference keys its table by config.json's `model_type` (tinyserve_llm/model/loader.py:22-25,
85-86); here `architectures[0]` is tried first and `model_type` second, with the same style of
error for an unknown one.
"""

from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Any, Callable, Mapping

from tinyserve_llm_amd.models.spec import ModelSpec


@dataclass(frozen=True)
class Architecture:
    name: str                                  # e.g. "LlamaForCausalLM"
    model_types: tuple[str, ...]               # config.json model_type values that also select it
    config_from_dict: Callable[[Mapping[str, Any]], Any]
    build_spec: Callable[[Any], ModelSpec]


ARCHITECTURES: dict[str, Architecture] = {}


def register_architecture(arch: Architecture) -> Architecture:
    ARCHITECTURES[arch.name] = arch
    return arch


def resolve(raw: Mapping[str, Any]) -> Architecture:
    for name in raw.get("architectures") or []:
        if name in ARCHITECTURES:
            return ARCHITECTURES[name]
    model_type = raw.get("model_type")
    for arch in ARCHITECTURES.values():
        if model_type in arch.model_types:
            return arch
    raise NotImplementedError(
        f"architecture {raw.get('architectures')!r} / model_type {model_type!r} is not supported; "
        f"have {sorted(ARCHITECTURES)}")


def read_config(folder: str) -> tuple[Architecture, Any]:
    """(architecture, typed configuration) of a model folder."""
    path = os.path.join(folder, "config.json")
    if not os.path.exists(path):
        raise FileNotFoundError(f"no config.json in {folder}")
    with open(path) as f:
        raw = json.load(f)
    arch = resolve(raw)
    return arch, arch.config_from_dict(raw)

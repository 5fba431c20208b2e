"""One registry from an architecture's name to its configuration class and its model builder.

The reference keys its table by config.json's `model_type` (tinyserve_llm/model/loader.py:22-25,
85-86); here `architectures[0]` is tried first and `model_type` second, with the same style of
error for an unknown one.
"""

from __future__ import annotations

import dataclasses
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
    # The way back, from a typed configuration to config.json's keys; None: the configuration's
    # fields under their own names (a dataclass's, else the object's attributes), which fits every
    # configuration class whose `from_dict` reads the keys it is made of.
    config_to_dict: Callable[[Any], Mapping[str, Any]] | None = None
    # The class of the typed configuration; None: the class whose classmethod `config_from_dict` is.
    config_type: type | None = None

    def owns(self, config: Any) -> bool:
        """Whether `config` is a typed configuration of this architecture."""
        kind = self.config_type or getattr(self.config_from_dict, "__self__", None)
        return isinstance(kind, type) and isinstance(config, kind)

    def to_dict(self, config: Any) -> dict[str, Any]:
        """config.json for `config`: its own keys, and the two by which `resolve` finds this
        architecture again if the configuration does not carry them."""
        if self.config_to_dict is not None:
            raw = dict(self.config_to_dict(config))
        elif dataclasses.is_dataclass(config):
            raw = dataclasses.asdict(config)
        else:
            raw = {k: v for k, v in vars(config).items() if not k.startswith("_")}
        if not raw.get("architectures"):
            raw["architectures"] = [self.name]
        if self.model_types and not raw.get("model_type"):
            raw["model_type"] = self.model_types[0]
        return raw


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


def architecture_of(config: Any) -> Architecture:
    """The architecture whose typed configuration `config` is."""
    for arch in ARCHITECTURES.values():
        if arch.owns(config):
            return arch
    raise NotImplementedError(f"no registered architecture has configurations of type {type(config).__name__}; "
                              f"have {sorted(ARCHITECTURES)}")


def write_config(folder: str, config: Any) -> str:
    """Writes `folder`/config.json for a typed configuration of a registered architecture."""
    os.makedirs(folder, exist_ok=True)
    path = os.path.join(folder, "config.json")
    with open(path, "w") as f:
        json.dump(architecture_of(config).to_dict(config), f, indent=1)
    return path


def read_config(folder: str) -> tuple[Architecture, Any]:
    """(architecture, typed configuration) of a model folder."""
    path = os.path.join(folder, "config.json")
    if not os.path.exists(path):
        raise FileNotFoundError(f"no config.json in {folder}")
    with open(path) as f:
        raw = json.load(f)
    arch = resolve(raw)
    return arch, arch.config_from_dict(raw)

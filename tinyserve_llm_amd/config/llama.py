"""Typed configuration of the Llama dense decoder, read from the keys of its config.json.

The reference reads the same keys ad hoc from an untyped transformers object
(tinyserve_llm/model/llama.py:86-104,193-197,219,232,260-268,294;
tinyserve_llm/engine/llm_engine.py:83,105-110). Here they are parsed once into a frozen
dataclass and validated; nothing downstream carries a size or constant of its own.
"""

from __future__ import annotations

import json
import os
from dataclasses import dataclass, asdict
from typing import Any, Mapping


class ConfigError(ValueError):
    """A config.json that this engine cannot run, with the offending key named."""


@dataclass(frozen=True)
class RopeScaling:
    """llama3 frequency scaling (tinyserve_llm/model/llama.py:107-128)."""

    factor: float
    low_freq_factor: float
    high_freq_factor: float
    original_max_position_embeddings: int


@dataclass(frozen=True)
class LlamaConfig:
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    max_position_embeddings: int
    rms_norm_eps: float
    rope_theta: float = 10000.0
    rope_scaling: RopeScaling | None = None
    tie_word_embeddings: bool = False
    eos_token_id: int = -1
    architecture: str = "LlamaForCausalLM"
    model_type: str = "llama"

    # ---- derived sizes -------------------------------------------------------------------
    @property
    def q_size(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_key_value_heads * self.head_dim

    @property
    def group_size(self) -> int:
        return self.num_attention_heads // self.num_key_value_heads

    # ---- parsing -------------------------------------------------------------------------
    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "LlamaConfig":
        def need(key: str) -> Any:
            if key not in raw or raw[key] is None:
                raise ConfigError(f"config.json lacks the required key {key!r}")
            return raw[key]

        for flag in ("attention_bias", "mlp_bias"):
            if raw.get(flag):
                raise ConfigError(f"{flag}=true is not supported: this decoder has no biases")
        act = raw.get("hidden_act", "silu")
        if act != "silu":
            raise ConfigError(f"hidden_act {act!r} is not supported; the gated MLP uses 'silu'")

        hidden = int(need("hidden_size"))
        heads = int(need("num_attention_heads"))
        kv_heads = int(raw.get("num_key_value_heads") or heads)
        head_dim = raw.get("head_dim") or hidden // heads
        theta, scaling = _rope_settings(raw)
        max_pos = int(need("max_position_embeddings"))
        if scaling is not None:
            scaling = RopeScaling(
                factor=float(_need_in(scaling, "factor")),
                low_freq_factor=float(_need_in(scaling, "low_freq_factor")),
                high_freq_factor=float(_need_in(scaling, "high_freq_factor")),
                original_max_position_embeddings=int(
                    scaling.get("original_max_position_embeddings", max_pos)),
            )
        eos = raw.get("eos_token_id", -1)
        if isinstance(eos, (list, tuple)):
            eos = eos[0] if eos else -1
        if eos is None:
            eos = -1
        archs = raw.get("architectures") or ["LlamaForCausalLM"]
        config = cls(
            vocab_size=int(need("vocab_size")),
            hidden_size=hidden,
            intermediate_size=int(need("intermediate_size")),
            num_hidden_layers=int(need("num_hidden_layers")),
            num_attention_heads=heads,
            num_key_value_heads=kv_heads,
            head_dim=int(head_dim),
            max_position_embeddings=max_pos,
            rms_norm_eps=float(need("rms_norm_eps")),
            rope_theta=theta,
            rope_scaling=scaling,
            tie_word_embeddings=bool(raw.get("tie_word_embeddings", False)),
            eos_token_id=int(eos),
            architecture=str(archs[0]),
            model_type=str(raw.get("model_type", "llama")),
        )
        config.validate()
        return config

    @classmethod
    def from_json(cls, path: str) -> "LlamaConfig":
        if os.path.isdir(path):
            path = os.path.join(path, "config.json")
        with open(path) as f:
            return cls.from_dict(json.load(f))

    def validate(self) -> None:
        positive = ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                    "num_attention_heads", "num_key_value_heads", "head_dim", "max_position_embeddings")
        for key in positive:
            if getattr(self, key) <= 0:
                raise ConfigError(f"{key} must be positive, got {getattr(self, key)}")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"num_attention_heads={self.num_attention_heads} is not a multiple of "
                f"num_key_value_heads={self.num_key_value_heads}")
        if self.head_dim % 2:
            raise ConfigError(f"head_dim={self.head_dim} must be even for rotate-half RoPE")
        if not self.rms_norm_eps > 0:
            raise ConfigError(f"rms_norm_eps must be positive, got {self.rms_norm_eps}")
        s = self.rope_scaling
        if s is not None and s.high_freq_factor == s.low_freq_factor:
            raise ConfigError("rope_scaling: high_freq_factor equals low_freq_factor")

    # ---- writing -------------------------------------------------------------------------
    def to_dict(self) -> dict[str, Any]:
        """config.json in the Hub's spelling: rope_theta and rope_scaling at the top level."""
        out = asdict(self)
        out["architectures"] = [out.pop("architecture")]
        out["hidden_act"] = "silu"
        out["attention_bias"] = False
        out["mlp_bias"] = False
        if self.rope_scaling is not None:
            out["rope_scaling"] = {"rope_type": "llama3", **asdict(self.rope_scaling)}
        return out

    def save(self, folder: str) -> None:
        os.makedirs(folder, exist_ok=True)
        with open(os.path.join(folder, "config.json"), "w") as f:
            json.dump(self.to_dict(), f, indent=1)


def _need_in(scaling: Mapping[str, Any], key: str) -> Any:
    if key not in scaling:
        raise ConfigError(f"rope_scaling lacks {key!r}")
    return scaling[key]


def _rope_settings(raw: Mapping[str, Any]) -> tuple[float, Mapping[str, Any] | None]:
    """Both spellings of the RoPE settings (tinyserve_llm/model/llama.py:86-104): a
    `rope_parameters` dict that also carries rope_theta, or top-level rope_theta + rope_scaling;
    `rope_type` or `type`; "default" means no scaling; anything but llama3 is refused."""
    params = raw.get("rope_parameters")
    if params:
        theta = params.get("rope_theta", raw.get("rope_theta", 10000.0))
        scaling = params
    else:
        theta = raw.get("rope_theta", 10000.0)
        scaling = raw.get("rope_scaling")
    if scaling is not None:
        rope_type = scaling.get("rope_type", scaling.get("type", "default"))
        if rope_type == "default":
            scaling = None
        elif rope_type != "llama3":
            raise NotImplementedError(f"rope_type {rope_type!r} is not supported")
    return float(theta), scaling

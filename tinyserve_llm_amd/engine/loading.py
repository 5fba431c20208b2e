"""From a model folder (or a configuration and a seed) to a model bound to its weights on the GPU."""

from __future__ import annotations

import torch

from tinyserve_llm_amd import models  # noqa: F401  (registers the architectures)
from tinyserve_llm_amd.models.decoder import DecoderModel
from tinyserve_llm_amd.models.registry import read_config, resolve
from tinyserve_llm_amd.weights.loader import load_params
from tinyserve_llm_amd.weights.random_init import random_params

DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32}


def as_dtype(dtype: str | torch.dtype) -> torch.dtype:
    if isinstance(dtype, torch.dtype):
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError(f"the engine runs in bfloat16 or float32, not {dtype}")
        return dtype
    try:
        return DTYPES[dtype]
    except KeyError:
        raise ValueError(f"dtype {dtype!r}: choose bfloat16 or float32") from None


def require_gpu(device: str | torch.device) -> torch.device:
    device = torch.device(device)
    if device.type != "cuda" or not torch.cuda.is_available():
        raise RuntimeError("this engine runs on an AMD GPU only (device 'cuda:N' under ROCm); "
                           "there is no CPU path")
    return device


def load_model(folder: str, dtype: str | torch.dtype = torch.bfloat16, device: str | torch.device = "cuda:0"
               ) -> tuple[DecoderModel, object]:
    """(model bound to the folder's weights, its typed configuration). The model class is chosen
    by config.json (tinyserve_llm/model/loader.py:73-95)."""
    device = require_gpu(device)
    dtype = as_dtype(dtype)
    arch, config = read_config(folder)
    model = DecoderModel(arch.build_spec(config))
    model.bind(load_params(model, folder, dtype, device), dtype, device)
    return model, config


def random_model(config, seed: int, dtype: str | torch.dtype = torch.bfloat16,
                 device: str | torch.device = "cuda:0") -> DecoderModel:
    """A model of `config` with weights drawn on the device from `seed` (no files)."""
    device = require_gpu(device)
    dtype = as_dtype(dtype)
    arch = resolve(config.to_dict())
    model = DecoderModel(arch.build_spec(config))
    model.bind(random_params(model, seed, dtype, device), dtype, device)
    return model

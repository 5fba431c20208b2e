"""From a model folder (or a configuration and a seed) to a model bound to its weights on the GPU."""

from __future__ import annotations

import torch

from tinyserve_llm_amd import models  # noqa: F401  (registers the architectures)
from tinyserve_llm_amd.models.decoder import DecoderModel
from tinyserve_llm_amd.models.registry import architecture_of, read_config
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


def streaming_copies(model: DecoderModel, policy: bool | None, device: torch.device) -> int:
    """Second copies of layer weights in the decode kernels' reading order (about a sixth faster
    to stream, for 60 % more weight memory at the 1B shape). `policy` None: only if the model's own
    weights take less than a fifth of the memory that is still free."""
    if policy is None:
        own = sum(p.numel() * p.element_size() for p in _bound_tensors(model))
        policy = model.dtype == torch.bfloat16 and own < torch.cuda.mem_get_info(device)[0] / 5
    return model.keep_streaming_copies() if policy else 0


def _bound_tensors(model: DecoderModel):
    """Every parameter tensor the model's parts hold (a tied head's is the embedding's: counted once)."""
    seen: set[int] = set()
    parts = [p for layer in model.layers for p in layer.parts().values()] + [model.embedding, model.head, model.final_norm]
    for part in parts:
        for name in part.param_specs():
            t = getattr(part, name, None)
            if isinstance(t, torch.Tensor) and t.data_ptr() not in seen:
                seen.add(t.data_ptr())
                yield t


def load_model(folder: str, dtype: str | torch.dtype = torch.bfloat16, device: str | torch.device = "cuda:0",
               keep_streaming_copies: bool | None = None) -> tuple[DecoderModel, object]:
    """(model bound to the folder's weights, its typed configuration). The model class is chosen
    by config.json (tinyserve_llm/model/loader.py:73-95)."""
    device = require_gpu(device)
    dtype = as_dtype(dtype)
    arch, config = read_config(folder)
    model = DecoderModel(arch.build_spec(config))
    model.bind(load_params(model, folder, dtype, device), dtype, device)
    streaming_copies(model, keep_streaming_copies, device)
    return model, config


def random_model(config, seed: int, dtype: str | torch.dtype = torch.bfloat16,
                 device: str | torch.device = "cuda:0", keep_streaming_copies: bool | None = None) -> DecoderModel:
    """A model of `config` with weights drawn on the device from `seed` (no files)."""
    device = require_gpu(device)
    dtype = as_dtype(dtype)
    arch = architecture_of(config)
    model = DecoderModel(arch.build_spec(config))
    model.bind(random_params(model, seed, dtype, device), dtype, device)
    streaming_copies(model, keep_streaming_copies, device)
    return model

"""From a model folder (or a configuration and a seed) to a model bound to its weights on the GPU."""

from __future__ import annotations

import logging

import torch

from tinyserve_llm_amd import models  # noqa: F401  (registers the architectures)
from tinyserve_llm_amd.models.decoder import DecoderModel
from tinyserve_llm_amd.models.registry import architecture_of, read_config
from tinyserve_llm_amd.weights.loader import load_params
from tinyserve_llm_amd.weights.random_init import random_params

logger = logging.getLogger(__name__)

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


STREAMING_COPIES_AT_MOST = 2.0     # times the weights' own bytes: a weight keeps at most one copy per kernel form
STREAMING_COPIES_SHARE = 0.25      # of the free memory that the weights' copies may take at most


def streaming_copies(model: DecoderModel, policy: bool | None, device: torch.device) -> int:
    """Second copies of the weights in the decode kernels' reading orders (about a sixth faster to
    stream). A weight keeps up to one copy per kernel form that can take it (16-row tiles, 8-row
    tiles, and for q|k|v the tiles regrouped for the rotation), so the copies come to between one and
    two times the weights' own bytes (1.9 times at the Llama 3.2 1B shape: every projection but q|k|v
    keeps both tile forms). `policy` None: made only
    if twice the weights' bytes are less than a quarter of the memory that is still free, which
    leaves the cache pool what it had; the bytes taken are logged. Returns the bytes taken."""
    if policy is None:
        own = sum(p.numel() * p.element_size() for p in _bound_tensors(model))
        free = torch.cuda.mem_get_info(device)[0]
        policy = model.dtype == torch.bfloat16 and STREAMING_COPIES_AT_MOST * own < STREAMING_COPIES_SHARE * free
    taken = model.keep_streaming_copies() if policy else 0
    if taken:
        logger.info("streaming copies of the weights: %.2f GB beside the weights' own bytes", taken / 1e9)
    return taken


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

"""Random-weights mode: parameters drawn from a seed, either straight onto a device or written out
as a model folder (config.json + model.safetensors) under the checkpoint's own tensor names.

The reference has no such mode; its tests build a random model with a library and save it
(tests/test_llama.py:55-80). Here every parameter is drawn in 32-bit from one seeded generator, in
the fixed order of the model's parameter list, as mean + std * N(0, 1) with the (mean, std) its
part declares, and then rounded to the stored type.
"""

from __future__ import annotations

import os

import torch
from safetensors.torch import save_file

from tinyserve_llm_amd.models.decoder import DecoderModel
from tinyserve_llm_amd.models.registry import architecture_of, write_config
from tinyserve_llm_amd.weights.loader import storage_dtype


def random_params(model: DecoderModel, seed: int, dtype: torch.dtype, device: torch.device | str = "cpu"
                  ) -> dict[str, torch.Tensor]:
    device = torch.device(device)
    gen = torch.Generator(device=device).manual_seed(seed)
    out = {}
    for name, ps in model.param_specs().items():
        store = storage_dtype(ps, dtype)
        if store == torch.int32:
            out[name] = torch.zeros(ps.shape, dtype=store, device=device)
            continue
        mean, std = ps.init
        t = torch.randn(ps.shape, generator=gen, device=device, dtype=torch.float32)
        out[name] = t.mul_(std).add_(mean).to(store)
    return out


def checkpoint_tensors(model: DecoderModel, params: dict[str, torch.Tensor]) -> dict[str, torch.Tensor]:
    """Parameters split back into the tensors of a checkpoint, by the architecture's table."""
    out = {}
    for name, dest in model.spec.checkpoint.items():
        t = dest.view(params[dest.param])
        out[name] = (t.t() if dest.transpose else t).detach().cpu().contiguous().clone()
    return out


def write_random_model(folder: str, config, seed: int, dtype: torch.dtype = torch.bfloat16) -> str:
    """Writes `folder`/config.json and `folder`/model.safetensors for `config` (a typed
    configuration of a registered architecture) with weights drawn from `seed`."""
    model = DecoderModel(architecture_of(config).build_spec(config))
    write_config(folder, config)
    params = random_params(model, seed, dtype, "cpu")
    save_file(checkpoint_tensors(model, params), os.path.join(folder, "model.safetensors"))
    return folder

"""Weights from safetensors, by tensor name, into the parameters a model declares.

Files are `model*.safetensors` in sorted order (tinyserve_llm/model/loader.py:33-35). Each
checkpoint tensor goes to the destination the architecture's table names for it (a whole
parameter, a row or column slice of a fused one, one matrix of a stack, possibly transposed;
the reference knows whole parameters and row slices, loader.py:49-60). Everything that is wrong with a
checkpoint is collected and raised once: tensors the model needs and did not get ("did not
fill", loader.py:63-70), tensors it has no place for, and shapes that do not fit.
"""

from __future__ import annotations

import os
from glob import glob

import torch
from safetensors import safe_open

from tinyserve_llm_amd.models.decoder import DecoderModel
from tinyserve_llm_amd.parts.base import ParamSpec


class WeightsError(ValueError):
    def __init__(self, missing: list[str], unexpected: list[str], wrong_shape: list[str]) -> None:
        self.missing, self.unexpected, self.wrong_shape = missing, unexpected, wrong_shape
        lines = []
        if missing:
            lines.append(f"checkpoint did not fill: {missing}")
        if unexpected:
            lines.append(f"unexpected tensors: {unexpected}")
        if wrong_shape:
            lines.append(f"wrong shapes: {wrong_shape}")
        super().__init__("; ".join(lines))


def storage_dtype(spec: ParamSpec, compute: torch.dtype) -> torch.dtype:
    return {"compute": compute, "float32": torch.float32, "int32": torch.int32}[spec.storage]


def checkpoint_files(folder: str) -> list[str]:
    files = sorted(glob(os.path.join(folder, "model*.safetensors")))
    if not files:
        raise FileNotFoundError(f"no model*.safetensors in {folder}")
    return files


def load_params(model: DecoderModel, folder: str, dtype: torch.dtype, device: torch.device | str
                ) -> dict[str, torch.Tensor]:
    """Reads the checkpoint into freshly allocated parameters on `device` and returns them by
    the model's own parameter names. Floating parameters take the engine's dtype unless their
    spec asks for 32-bit; integer tables are int32."""
    spec = model.spec
    specs = model.param_specs()
    host: dict[str, torch.Tensor] = {
        name: torch.empty(ps.shape, dtype=storage_dtype(ps, dtype)) for name, ps in specs.items()}
    filled: dict[str, int] = {name: 0 for name in specs}       # elements written per parameter
    seen: set[str] = set()
    unexpected: list[str] = []
    wrong: list[str] = []
    for file in checkpoint_files(folder):
        with safe_open(file, "pt", "cpu") as f:
            for name in f.keys():
                if name.endswith(spec.ignored_suffixes) if spec.ignored_suffixes else False:
                    continue
                dest = spec.checkpoint.get(name)
                if dest is None:
                    if name not in spec.optional:
                        unexpected.append(name)
                    continue
                if name in seen:
                    wrong.append(f"{name}: present in more than one file")
                    continue
                seen.add(name)
                place = dest.view(host[dest.param])          # what of the parameter this tensor fills
                want = tuple(reversed(place.shape)) if dest.transpose else tuple(place.shape)
                got = tuple(f.get_slice(name).get_shape())
                if got != want:
                    wrong.append(f"{name}: checkpoint {list(got)}, model {list(want)}")
                    continue
                tensor = f.get_tensor(name)
                place.copy_(tensor.t() if dest.transpose else tensor)
                filled[dest.param] += place.numel()
    missing = sorted(n for n, d in spec.checkpoint.items() if n not in seen)
    # a parameter no checkpoint name maps to cannot be filled at all: that is a bug of the table
    unmapped = sorted(p for p, n in filled.items() if n != host[p].numel()
                      and not any(d.param == p for d in spec.checkpoint.values()))
    if unmapped:
        missing += [f"{p} (no checkpoint name maps to it)" for p in unmapped]
    if missing or unexpected or wrong:
        raise WeightsError(missing, sorted(unexpected), wrong)
    return {name: t.to(device) for name, t in host.items()}

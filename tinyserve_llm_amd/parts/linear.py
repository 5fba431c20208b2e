"""y = x · Wᵀ for bias-free projections stored [out, in] (tinyserve_llm/model/llama.py:179,201,221,293).

float32 runs the engine's own exact kernel (32-bit multiply-adds, ascending k, independent of the
batch). bfloat16 uses the skinny weight-streaming kernel for few rows and the vendor matrix
library for many, as the reference uses a vendor library for every projection.
"""

from __future__ import annotations

import torch

from tinyserve_llm_amd.ops import hip


def linear(x: torch.Tensor, weight: torch.Tensor, out_dtype: torch.dtype | None = None) -> torch.Tensor:
    if x.dtype == torch.float32:
        return hip.gemm_exact(x, weight, out_dtype)
    if x.dtype != torch.bfloat16:
        raise hip.KernelError(f"linear: no path for {x.dtype}")
    if not x.is_cuda:
        raise hip.KernelError("linear: GPU tensors only; there is no CPU path")
    return hip.linear_bf16(x, weight, out_dtype or torch.bfloat16)

"""RMSNorm with the residual add folded in (tinyserve_llm/model/llama.py:39-74).

`norm(x, residual)` returns (normalise(x + residual) * weight, x + residual): the sum, its mean
square, the rsqrt and the scaling are 32-bit; the returned residual is the sum rounded to the
storage type, while the normalisation uses the unrounded sum (llama.py:63-67).
"""

from __future__ import annotations

import torch

from tinyserve_llm_amd.ops import hip
from tinyserve_llm_amd.parts.base import Norm, ParamSpec, register
from tinyserve_llm_amd.parts.linear import DeferredNorm, NormRequest


@register("norm", "rmsnorm")
class RMSNorm(Norm):
    graph_safe = True

    def __init__(self, hidden_size: int, eps: float) -> None:
        self.hidden_size = hidden_size
        self.eps = eps
        self.weight: torch.Tensor | None = None

    def param_specs(self) -> dict[str, ParamSpec]:
        return {"weight": ParamSpec((self.hidden_size,), init=(1.0, 0.1))}

    def __call__(self, x, residual=None, rows=None):
        return hip.rmsnorm(x, self.weight, self.eps, residual, rows)

    def defer(self, x, residual=None) -> DeferredNorm:
        """The same norm as an operand that the next projection may fuse."""
        return DeferredNorm(x, residual, self.weight, self.eps)

    def request(self, residual=None) -> NormRequest:
        """The same norm as a request to the projection before it (`linear(..., then=)`)."""
        return NormRequest(self.weight, self.eps, residual)

    def made_for(self, pending) -> bool:
        """Whether `pending` is this norm, deferred (by `defer` or through `request`)."""
        return isinstance(pending, DeferredNorm) and pending.weight is self.weight and pending.eps == self.eps

"""SiLU-gated feed-forward (tinyserve_llm/model/llama.py:77-83,215-225): one fused projection gives
[gate | up], then silu(gate) * up, then the down projection."""

from __future__ import annotations

import torch

from tinyserve_llm_amd.parts.base import FeedForward, ParamSpec, StepContext, register
from tinyserve_llm_amd.parts.linear import linear, streaming_copy


@register("feed_forward", "gated_mlp")
class GatedMLP(FeedForward):
    graph_safe = True
    takes_deferred_norm = True
    finishes_into_norm = True

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "silu") -> None:
        if activation != "silu":
            raise ValueError(f"activation {activation!r}: the gated feed-forward kernel computes silu")
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.gate_up: torch.Tensor | None = None
        self.down: torch.Tensor | None = None
        self.gate_up_packed = None       # `streaming_copy` of each weight, if the model keeps them
        self.down_packed = None

    def param_specs(self) -> dict[str, ParamSpec]:
        return {"gate_up": ParamSpec((2 * self.intermediate_size, self.hidden_size)),
                "down": ParamSpec((self.hidden_size, self.intermediate_size))}

    def keep_streaming_copies(self) -> int:
        self.gate_up_packed, self.down_packed = streaming_copy(self.gate_up), streaming_copy(self.down)
        return sum(c.nbytes() for c in (self.gate_up_packed, self.down_packed) if c is not None)

    def forward(self, x: torch.Tensor, ctx: StepContext, then=None) -> torch.Tensor:
        gated = linear(x, self.gate_up, glu=True, packed=self.gate_up_packed, feeds=self.down)
        return linear(gated, self.down, packed=self.down_packed, then=then)

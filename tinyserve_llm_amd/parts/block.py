"""Arrangements of a layer's parts. "pre_norm" is the Llama block with the residual add deferred
into the next norm (tinyserve_llm/model/llama.py:238-253): a layer returns (feed-forward output,
residual) without adding them; the following norm adds. It equals h += mixer(norm(h));
h += feed_forward(norm(h))."""

from __future__ import annotations

from dataclasses import dataclass

import torch

from tinyserve_llm_amd.parts.base import FeedForward, LayerMemory, Mixer, Norm, StepContext, register


@dataclass
class Layer:
    mixer: Mixer
    feed_forward: FeedForward
    mixer_norm: Norm
    ff_norm: Norm
    block: str = "pre_norm"

    def parts(self) -> dict[str, object]:
        return {"mixer": self.mixer, "ff": self.feed_forward, "mixer_norm": self.mixer_norm, "ff_norm": self.ff_norm}


@register("block", "pre_norm")
def pre_norm_block(layer: Layer, hidden: torch.Tensor, residual: torch.Tensor | None, ctx: StepContext,
                   mem: LayerMemory) -> tuple[torch.Tensor, torch.Tensor]:
    pending = layer.mixer_norm.defer(hidden, residual) if layer.mixer.takes_deferred_norm else None
    if pending is None:
        x, residual = layer.mixer_norm(hidden, residual)
        x = layer.mixer.forward(x, ctx, mem)
    else:
        x = layer.mixer.forward(pending, ctx, mem)
        residual = pending.residual_out
    pending = layer.ff_norm.defer(x, residual) if layer.feed_forward.takes_deferred_norm else None
    if pending is None:
        x, residual = layer.ff_norm(x, residual)
        x = layer.feed_forward.forward(x, ctx)
    else:
        x = layer.feed_forward.forward(pending, ctx)
        residual = pending.residual_out
    return x, residual

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
    norms: dict[str, Norm]           # by the names the arrangement uses
    block: str = "pre_norm"

    def parts(self) -> dict[str, object]:
        """Every part by the name its parameters are known under (`layers.<i>.<name>.<parameter>`)."""
        if {"mixer", "ff"} & set(self.norms):
            raise ValueError("a norm cannot be named 'mixer' or 'ff'")
        return {"mixer": self.mixer, "ff": self.feed_forward, **self.norms}


def uses_norms(*names: str):
    """Declares the norms an arrangement looks up in `layer.norms`, so that a layer that lacks one
    is refused when the model is built, not at its first step."""
    def mark(fn):
        fn.norm_names = names
        return fn
    return mark


@register("block", "pre_norm")
@uses_norms("mixer_norm", "ff_norm")
def pre_norm_block(layer: Layer, hidden: torch.Tensor, residual: torch.Tensor | None, ctx: StepContext,
                   mem: LayerMemory) -> tuple[torch.Tensor, torch.Tensor]:
    mixer_norm, ff_norm = layer.norms["mixer_norm"], layer.norms["ff_norm"]
    pending = mixer_norm.defer(hidden, residual) if layer.mixer.takes_deferred_norm else None
    if pending is None:
        x, residual = mixer_norm(hidden, residual)
        x = layer.mixer.forward(x, ctx, mem)
    else:
        x = layer.mixer.forward(pending, ctx, mem)
        residual = pending.residual_out
    pending = ff_norm.defer(x, residual) if layer.feed_forward.takes_deferred_norm else None
    if pending is None:
        x, residual = ff_norm(x, residual)
        x = layer.feed_forward.forward(x, ctx)
    else:
        x = layer.feed_forward.forward(pending, ctx)
        residual = pending.residual_out
    return x, residual

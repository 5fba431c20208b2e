"""Arrangements of a layer's parts. "pre_norm" is the Llama block with the residual add deferred
into the next norm (tinyserve_llm/model/llama.py:238-253): a layer returns (feed-forward output,
residual) without adding them; the following norm adds. It equals h += mixer(norm(h));
h += feed_forward(norm(h)).

Norms travel between parts in two directions. Forward: a norm hands its input, deferred, to the
part after it, whose first projection fuses it (`Norm.defer`, `takes_deferred_norm`). Backward: a
norm asks the part before it to finish into it (`Norm.request`, `finishes_into_norm`): that part's
last projection then leaves the residual sum and half of the norm, and what the part returns is the
norm deferred, for the part after it. Between layers the model does the asking: it tells a block
which norm the next block starts with (`following=`), and a block that `starts_with` a norm accepts
that norm, deferred, as its `hidden` (with `residual` None: the sum is inside)."""

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


def starts_with(name: str):
    """Declares that an arrangement applies the norm of this name to (hidden, residual) before
    anything else, takes `following=` (the norm the next arrangement starts with, or None), and
    accepts its own first norm in deferred form as `hidden`."""
    def mark(fn):
        fn.first_norm = name
        return fn
    return mark


def first_norm_of(layer: Layer) -> Norm | None:
    """The norm a layer's arrangement starts with, if it says so (`starts_with`)."""
    from tinyserve_llm_amd.parts.base import BLOCKS
    name = getattr(BLOCKS[layer.block], "first_norm", None)
    return layer.norms[name] if name else None


def _through(part, norm: Norm, x, residual, run, following: Norm | None):
    """One branch of a pre-norm arrangement: `norm` applied to (x, residual), then `part` (`run` calls
    its forward). `x` may be `norm` itself in deferred form (then `residual` is None). The norm is
    handed to the part deferred if the part takes it so; the part is asked to finish into
    `following` if it can and that norm takes requests. Returns (the part's output or `following`
    deferred, the residual stream after `norm`'s sum)."""
    pending = x if norm.made_for(x) else None
    if pending is None and part.takes_deferred_norm:
        pending = norm.defer(x, residual)
    if pending is not None and not part.takes_deferred_norm:
        x, residual, pending = pending.materialize(), pending.residual_out, None
    elif pending is None:
        x, residual = norm(x, residual)
    # the stream after this norm's sum: known now, or once the part's first projection has run
    request = following.request(pending if pending is not None else residual) \
        if following is not None and part.finishes_into_norm else None
    out = run(pending if pending is not None else x, request) if request is not None else run(pending if pending is not None else x)
    if pending is not None:
        residual = pending.residual_out
    return out, residual


@register("block", "pre_norm")
@uses_norms("mixer_norm", "ff_norm")
@starts_with("mixer_norm")
def pre_norm_block(layer: Layer, hidden, residual: torch.Tensor | None, ctx: StepContext, mem: LayerMemory,
                   following: Norm | None = None) -> tuple[torch.Tensor, torch.Tensor | None]:
    mixer_norm, ff_norm = layer.norms["mixer_norm"], layer.norms["ff_norm"]
    x, residual = _through(layer.mixer, mixer_norm, hidden, residual,
                           lambda x, then=None: layer.mixer.forward(x, ctx, mem, **({"then": then} if then else {})), ff_norm)
    if ff_norm.made_for(x):
        residual = None                      # the sum is inside the deferred norm
    x, residual = _through(layer.feed_forward, ff_norm, x, residual,
                           lambda x, then=None: layer.feed_forward.forward(x, ctx, **({"then": then} if then else {})), following)
    if following is not None and following.made_for(x):
        residual = None
    return x, residual

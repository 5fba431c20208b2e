"""A model as data: which parts make each layer, in which order layers run, whose cache each run
uses, and where every checkpoint tensor goes. An architecture is a function from its typed
configuration to a ModelSpec; the generic decoder (models/decoder.py) runs any ModelSpec."""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Mapping

from tinyserve_llm_amd.parts.base import PartSpec


@dataclass(frozen=True)
class LayerSpec:
    """The parts of one layer: a mixer, a feed-forward, and the norms that its block arrangement
    asks for, by the names it asks for them under ("mixer_norm" and "ff_norm" for "pre_norm"; an
    arrangement with norms after its parts, or with one norm for two branches, names its own)."""

    mixer: PartSpec
    feed_forward: PartSpec
    norms: Mapping[str, PartSpec]
    block: str = "pre_norm"

    @classmethod
    def pre_norm(cls, mixer: PartSpec, feed_forward: PartSpec, mixer_norm: PartSpec, ff_norm: PartSpec) -> "LayerSpec":
        return cls(mixer, feed_forward, {"mixer_norm": mixer_norm, "ff_norm": ff_norm}, "pre_norm")


@dataclass(frozen=True)
class LayerRun:
    """One entry of the run order. `layer` indexes ModelSpec.layers (a layer may be named twice:
    same weights, run again). `cache` names the cache this run uses: None = a cache of its own;
    an int = the cache of that earlier entry of the order, which this run reads and, unless `store`
    is False, also writes."""

    layer: int
    cache: int | None = None
    store: bool = True


@dataclass(frozen=True)
class Destination:
    """Where a checkpoint tensor lands: in parameter `param`, or in the slice `param[index]` of a
    parameter that stacks several matrices (experts, say); there in rows [row, row + rows) and, for
    matrices, columns [col, col + cols) (None = all of them); `transpose`: the checkpoint stores
    the matrix the other way round."""

    param: str
    row: int = 0
    rows: int | None = None
    col: int = 0
    cols: int | None = None
    transpose: bool = False
    index: tuple[int, ...] = ()

    def view(self, param):
        """The part of `param` (a tensor) that the checkpoint tensor fills, as a view."""
        t = param[self.index] if self.index else param
        t = t.narrow(0, self.row, self.rows if self.rows is not None else t.shape[0] - self.row)
        if t.dim() > 1:
            t = t.narrow(1, self.col, self.cols if self.cols is not None else t.shape[1] - self.col)
        elif self.col or self.cols is not None:
            raise ValueError(f"{self.param} has no columns to slice")
        return t


@dataclass
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden_size: int
    max_position: int | None          # None: the model's parts set no limit to a request's length
    layers: list[LayerSpec]
    order: list[LayerRun]
    final_norm: PartSpec
    position_encodings: dict[str, PartSpec] = field(default_factory=dict)
    tie_word_embeddings: bool = False
    eos_token_id: int = -1
    embedding_init: tuple[float, float] = (0.0, 0.02)
    # what turns token ids into the first hidden rows, and the final rows into logits; None: a
    # plain table and a plain projection (tied to the table if `tie_word_embeddings`)
    embedding: PartSpec | None = None
    head: PartSpec | None = None
    # checkpoint tensor name -> destination; names matching `ignored_suffixes` are skipped
    checkpoint: dict[str, Destination] = field(default_factory=dict)
    ignored_suffixes: tuple[str, ...] = ()
    # tensors that may be present but are not needed (a tied checkpoint's copy of the embedding)
    optional: tuple[str, ...] = ()

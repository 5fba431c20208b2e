"""A model as data: which parts make each layer, in which order layers run, whose cache each run
uses, and where every checkpoint tensor goes. An architecture is a function from its typed
configuration to a ModelSpec; the generic decoder (models/decoder.py) runs any ModelSpec."""

from __future__ import annotations

from dataclasses import dataclass, field

from tinyserve_llm_amd.parts.base import PartSpec


@dataclass(frozen=True)
class LayerSpec:
    mixer: PartSpec
    feed_forward: PartSpec
    mixer_norm: PartSpec
    ff_norm: PartSpec
    block: str = "pre_norm"


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
    """Where a checkpoint tensor lands: rows [row, row + rows) of parameter `param`
    (rows None = the whole parameter)."""

    param: str
    row: int = 0
    rows: int | None = None


@dataclass
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden_size: int
    max_position: int
    layers: list[LayerSpec]
    order: list[LayerRun]
    final_norm: PartSpec
    position_encodings: dict[str, PartSpec] = field(default_factory=dict)
    tie_word_embeddings: bool = False
    eos_token_id: int = -1
    embedding_init: tuple[float, float] = (0.0, 0.02)
    # checkpoint tensor name -> destination; names matching `ignored_suffixes` are skipped
    checkpoint: dict[str, Destination] = field(default_factory=dict)
    ignored_suffixes: tuple[str, ...] = ()
    # tensors that may be present but are not needed (a tied checkpoint's copy of the embedding)
    optional: tuple[str, ...] = ()

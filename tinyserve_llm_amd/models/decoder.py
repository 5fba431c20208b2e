"""The generic decoder: builds the parts a ModelSpec names, owns their parameters, and runs the
layers in the order the spec lists over one packed step (tinyserve_llm/model/llama.py:256-304 is
the fixed-architecture counterpart). Nothing here is specific to one architecture."""

from __future__ import annotations

from dataclasses import dataclass

import torch

from tinyserve_llm_amd.models.spec import ModelSpec
from tinyserve_llm_amd.parts import base
from tinyserve_llm_amd.parts.base import KVSpec, LayerMemory, ParamSpec, PartSpec, StateSpec, StepContext
from tinyserve_llm_amd.parts.block import Layer, first_norm_of


@dataclass(frozen=True)
class CachePlanEntry:
    """One cache of the model: which run of the order owns it and what its mixer stores."""

    owner: int          # index into ModelSpec.order of the run that owns (first writes) it
    kv: KVSpec


@dataclass(frozen=True)
class StatePlanEntry:
    run: int            # index into ModelSpec.order
    state: StateSpec


class DecoderModel:
    def __init__(self, spec: ModelSpec) -> None:
        self.spec = spec
        self.layers: list[Layer] = []
        for ls in spec.layers:
            # one LayerSpec object listed at several indices still gives one set of weights per index
            if ls.block not in base.BLOCKS:
                raise KeyError(f"no block arrangement named {ls.block!r}; registered: {sorted(base.BLOCKS)}")
            lacking = [n for n in getattr(base.BLOCKS[ls.block], "norm_names", ()) if n not in ls.norms]
            if lacking:
                raise KeyError(f"block arrangement {ls.block!r} asks for the norms {lacking}; the layer names {sorted(ls.norms)}")
            self.layers.append(Layer(
                mixer=base.make("mixer", ls.mixer), feed_forward=base.make("feed_forward", ls.feed_forward),
                norms={name: base.make("norm", ps) for name, ps in ls.norms.items()}, block=ls.block))
        self.final_norm = base.make("norm", spec.final_norm)
        self.position_encodings = {name: base.make("position_encoding", ps)
                                   for name, ps in spec.position_encodings.items()}
        sizes = dict(vocab_size=spec.vocab_size, hidden_size=spec.hidden_size, init=spec.embedding_init)
        self.embedding = base.make("embedding", spec.embedding or PartSpec("table", sizes))
        self.head = base.make("head", spec.head or PartSpec("projection", dict(sizes, tied=spec.tie_word_embeddings)))
        self.dtype: torch.dtype | None = None
        self.device: torch.device | None = None
        self._check_order()

    # ---- structure ---------------------------------------------------------------------------
    def _check_order(self) -> None:
        for i, run in enumerate(self.spec.order):
            if not 0 <= run.layer < len(self.layers):
                raise ValueError(f"order[{i}] names layer {run.layer}, the model has {len(self.layers)}")
            if run.cache is not None:
                if not 0 <= run.cache < i:
                    raise ValueError(f"order[{i}] uses the cache of entry {run.cache}, which does not run before it")
                owner = self.spec.order[run.cache]
                if owner.cache is not None:
                    raise ValueError(f"order[{i}] must name the entry that owns the cache, not a borrower")
                a, b = self.layers[run.layer].mixer.kv_spec(), self.layers[owner.layer].mixer.kv_spec()
                if a is None or b is None or (a.num_kv_heads, a.head_dim) != (b.num_kv_heads, b.head_dim):
                    raise ValueError(f"order[{i}] and order[{run.cache}] cache rows of different shapes")
            elif not run.store and self.layers[run.layer].mixer.kv_spec() is not None:
                raise ValueError(f"order[{i}] neither owns a cache to write nor names one to read")

    def cache_plan(self) -> list[CachePlanEntry]:
        """The caches the model needs, in run order; a run that borrows adds none."""
        plan = []
        for i, run in enumerate(self.spec.order):
            kv = self.layers[run.layer].mixer.kv_spec()
            if kv is not None and run.cache is None:
                plan.append(CachePlanEntry(i, kv))
        return plan

    def state_plan(self) -> list[StatePlanEntry]:
        plan = []
        for i, run in enumerate(self.spec.order):
            st = self.layers[run.layer].mixer.state_spec()
            if st is not None:
                plan.append(StatePlanEntry(i, st))
        return plan

    def graph_safe(self) -> bool:
        """True if every part may be recorded into a HIP graph (see Part.graph_safe)."""
        parts = [p for layer in self.layers for p in layer.parts().values()]
        parts += [self.final_norm, self.embedding, self.head, *self.position_encodings.values()]
        return all(getattr(p, "graph_safe", False) for p in parts)

    # ---- parameters --------------------------------------------------------------------------
    def param_specs(self) -> dict[str, ParamSpec]:
        out: dict[str, ParamSpec] = {f"embed.{pname}": ps for pname, ps in self.embedding.param_specs().items()}
        for i, layer in enumerate(self.layers):
            for part_name, part in layer.parts().items():
                for pname, ps in part.param_specs().items():
                    out[f"layers.{i}.{part_name}.{pname}"] = ps
        for name, enc in self.position_encodings.items():
            for pname, ps in enc.param_specs().items():
                out[f"positions.{name}.{pname}"] = ps
        for pname, ps in self.final_norm.param_specs().items():
            out[f"final_norm.{pname}"] = ps
        for pname, ps in self.head.param_specs().items():
            out[f"head.{pname}"] = ps
        return out

    def bind(self, params: dict[str, torch.Tensor], dtype: torch.dtype, device: torch.device) -> None:
        """Hand every part its parameters (already on the device, in their storage types)."""
        self.dtype, self.device = dtype, device
        grouped: dict[str, dict[str, torch.Tensor]] = {}
        for name, tensor in params.items():
            owner, _, pname = name.rpartition(".")
            grouped.setdefault(owner, {})[pname] = tensor
        self.embedding.bind(grouped.get("embed", {}))
        self.head.bind(grouped.get("head", {}))
        if self.spec.tie_word_embeddings:
            self.head.tie(self.embedding.table())
        for i, layer in enumerate(self.layers):
            for part_name, part in layer.parts().items():
                part.bind(grouped.get(f"layers.{i}.{part_name}", {}))
        for name, enc in self.position_encodings.items():
            enc.bind(grouped.get(f"positions.{name}", {}))
            enc.prepare(device)
        self.final_norm.bind(grouped.get("final_norm", {}))

    def widest_activation(self) -> int:
        """Elements per token of the widest tensor any layer makes (the parts say: `Part.widest_activation`)."""
        return max([self.spec.hidden_size] + [part.widest_activation() for layer in self.layers
                                              for part in layer.parts().values()])

    def keep_streaming_copies(self) -> int:
        """Lets every part of every layer keep its weights once more in a decode kernel's reading
        order, and the head likewise; returns the bytes that takes."""
        return self.head.keep_streaming_copies() + sum(part.keep_streaming_copies() for layer in self.layers
                                                       for part in layer.parts().values())

    # ---- one step ----------------------------------------------------------------------------
    def forward(self, ctx: StepContext, memory: list[LayerMemory]) -> tuple[torch.Tensor, torch.Tensor | None]:
        """Runs the step's tokens through every entry of the order; returns the last feed-forward
        output and the residual stream, whose sum the final norm takes."""
        ctx.position_encodings = self.position_encodings
        hidden = self.embedding.forward(ctx)
        for enc in self.position_encodings.values():
            hidden = enc.on_embedding(hidden, ctx)
        residual = None
        order = self.spec.order
        for i, (run, mem) in enumerate(zip(order, memory)):
            layer = self.layers[run.layer]
            block = base.BLOCKS[layer.block]
            if getattr(block, "first_norm", None) is None:
                hidden, residual = block(layer, hidden, residual, ctx, mem)
                continue
            # the norm the next run starts with, which this one's last projection may finish into
            # (after the last run comes the final norm, which picks rows: it takes plain tensors)
            following = first_norm_of(self.layers[order[i + 1].layer]) if i + 1 < len(order) else None
            hidden, residual = block(layer, hidden, residual, ctx, mem, following=following)
        return hidden, residual

    def logits(self, hidden: torch.Tensor, residual: torch.Tensor | None, rows: torch.Tensor) -> torch.Tensor:
        """float32 logits [len(rows), vocab] at the wanted rows only: the final norm and the
        vocabulary projection touch no other row (tinyserve_llm/engine/model_runner.py:125-127)."""
        normed, _ = self.final_norm(hidden, residual, rows)
        return self.head.forward(normed)

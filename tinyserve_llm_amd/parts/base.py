"""What a part of a layer is, and the registries that a configuration picks parts from.

A layer is assembled from a mixer, a feed-forward and the norms its arrangement (a block) names;
position encodings are shared parts that mixers refer to by name; an embedding and a head stand
at the two ends of the model. Each part is built
from explicit sizes and constants, declares the parameters it needs, receives them once, and then
works on flat batches of tokens. No part knows which model or which layer it is in.

The reference passes its config object into attention and decoder layer
(tinyserve_llm/model/llama.py:191,230) and hands attention an injected backend
(tinyserve_llm/model/attention.py:13-26); here the seam is wider: every kind of part sits behind an
interface and a name, so that one model may use different mixers and feed-forwards layer by layer.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable

import torch


# ---- declarations ---------------------------------------------------------------------------

@dataclass(frozen=True)
class ParamSpec:
    """One parameter of a part. `storage`: "compute" = the engine's dtype (bfloat16 or float32),
    "float32" = kept in 32-bit whatever the engine's dtype, "int32" = an integer table.
    `init` = (mean, std) of the normal distribution that the random-weights mode draws from."""

    shape: tuple[int, ...]
    storage: str = "compute"
    init: tuple[float, float] = (0.0, 0.02)


@dataclass(frozen=True)
class KVSpec:
    """A mixer that caches a key and a value row per token. `window` 0 = every key is kept;
    W > 0 = only the last W positions are ever read, so older pages can be given back."""

    num_kv_heads: int
    head_dim: int
    window: int = 0


@dataclass(frozen=True)
class StateSpec:
    """Fixed-size state that a mixer keeps per request (one slot per live request)."""

    shape: tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass
class LayerMemory:
    """What one run of a layer may touch of the engine's memory."""

    k_cache: torch.Tensor | None = None   # [pages, page_size, kv_heads, head_dim] view of this run's cache
    v_cache: torch.Tensor | None = None
    space: int = 0                        # which page space's block tables and slots address it
    store: bool = True                    # False: read another run's cache, write nothing
    state: torch.Tensor | None = None     # [slots, *StateSpec.shape]


@dataclass
class StepContext:
    """One step's batch, packed: tokens of several requests back to back, portions of prompts
    beside single decoded tokens. Index tensors live on the device; the lists mirror them on the
    host. `slot_mapping[s]` and `block_tables[s]` belong to page space s."""

    num_tokens: int
    num_seqs: int
    token_ids: torch.Tensor               # [T] int32
    positions: torch.Tensor               # [T] int32, absolute position of each token in its request
    seq_of_token: torch.Tensor            # [T] int32, row of the batch each token belongs to
    cu_seqlens: torch.Tensor              # [S+1] int32
    context_lens: torch.Tensor            # [S] int32, keys of each request after this step's writes
    state_slots: torch.Tensor             # [S] int32
    slot_mapping: list[torch.Tensor]      # per space: [T] int32, page * page_size + offset
    block_tables: list[torch.Tensor]      # per space: [S, max_pages] int32, in pages of `page_size` tokens
    host_cu_seqlens: list[int] = field(default_factory=list)
    host_starts: list[int] = field(default_factory=list)      # first position fed, per request
    host_context_lens: list[int] = field(default_factory=list)
    host_state_slots: list[int] = field(default_factory=list)
    position_encodings: dict[str, "PositionEncoding"] = field(default_factory=dict)
    scratch: dict = field(default_factory=dict)     # what parts derive from a step once and share
    page_size: int = 0                    # tokens per entry of the block tables (0: a page of the cache views; the pools may
                                          # be cut into shorter pages, entry e then standing for the consecutive pages e n + j)

    @property
    def max_query_len(self) -> int:
        c = self.host_cu_seqlens
        return max((b - a for a, b in zip(c, c[1:])), default=0)


# ---- interfaces -----------------------------------------------------------------------------

class Part:
    """Base of every part: declares parameters, receives them."""

    # True if forward() only launches work on the current stream from the device tensors of the
    # step context (no host reads of them, no Python branching on the host lists): such a part
    # can be recorded into a HIP graph and replayed with new inputs.
    graph_safe = False

    def param_specs(self) -> dict[str, ParamSpec]:
        return {}

    def bind(self, params: dict[str, torch.Tensor]) -> None:
        for name, tensor in params.items():
            setattr(self, name, tensor)

    def widest_activation(self) -> int:
        """Elements per token of the widest tensor the part makes on its way: the engine sets memory
        aside for a step's activations by it. The default is the most rows of any of the part's
        matrices (a projection's output; the last two dimensions of stacked matrices count)."""
        return max((ps.shape[-2] for ps in self.param_specs().values() if len(ps.shape) >= 2), default=0)

    def keep_streaming_copies(self) -> int:
        """Optionally keeps second copies of weights in the order a decode kernel reads them
        (`parts.linear.streaming_copy`), to hand to `linear(..., packed=)`; returns the bytes they
        take. Called after `bind` when memory allows. The default keeps none."""
        return 0


class Norm(Part):
    def __call__(self, x: torch.Tensor, residual: torch.Tensor | None = None,
                 rows: torch.Tensor | None = None) -> tuple[torch.Tensor, torch.Tensor | None]:
        """(normalised(x + residual), x + residual); `rows` restricts the output to some rows."""
        raise NotImplementedError

    def defer(self, x: torch.Tensor, residual: torch.Tensor | None = None):
        """Optionally the norm as an operand for a part that declares `takes_deferred_norm`: an
        object whose first consumer computes it (possibly fused into its own kernel) and which
        then holds `residual_out`. None (the default): this norm is always computed by itself."""
        return None

    def request(self, residual=None):
        """Optionally the norm as a request to the part before it, if that part declares
        `finishes_into_norm`: the part hands the request to its last projection (`then=`) and returns
        what comes back, this norm deferred with its first half done. `residual` is the stream the
        part's output is added to (a tensor, None, or a deferred norm that will hold it). None (the
        default): this norm takes plain tensors only."""
        return None

    def made_for(self, pending) -> bool:
        """Whether `pending` is this very norm in deferred form."""
        return False


class PositionEncoding(Part):
    def prepare(self, device: torch.device) -> None:
        """Build tables on the device (called once, after bind)."""

    def rotary_table(self) -> torch.Tensor | None:
        """float32 [positions, head_dim] = [cos | sin] for rotate-half mixers, or None."""
        return None

    def on_embedding(self, hidden: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        """Hook for encodings that act on the embedded tokens."""
        return hidden


class Mixer(Part):
    # True if forward() passes x to exactly one `linear()` call and uses it nowhere else, so that a
    # norm may hand it over deferred (see Norm.defer)
    takes_deferred_norm = False
    # True if forward() takes `then=` (a request of the norm that follows: Norm.request), hands it to
    # the `linear()` call that makes its result, and returns what that call returns
    finishes_into_norm = False

    def kv_spec(self) -> KVSpec | None:
        return None

    def state_spec(self) -> StateSpec | None:
        return None

    def forward(self, x: torch.Tensor, ctx: StepContext, mem: LayerMemory) -> torch.Tensor:
        raise NotImplementedError


class FeedForward(Part):
    takes_deferred_norm = False    # as for Mixer
    finishes_into_norm = False     # as for Mixer

    def forward(self, x: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        raise NotImplementedError


class Embedding(Part):
    """Token ids to the first hidden rows [tokens, hidden]."""

    def forward(self, ctx: StepContext) -> torch.Tensor:
        raise NotImplementedError

    def table(self) -> torch.Tensor | None:
        """The [vocab, hidden] matrix a tied head may share, or None if there is none to share."""
        return None


class Head(Part):
    """The final (already normalised) rows to float32 logits [rows, vocab]."""

    def tie(self, table: torch.Tensor) -> None:
        """Called instead of handing the head a weight of its own when the model ties it to the embedding."""
        raise NotImplementedError(f"{type(self).__name__} cannot be tied to the embedding")

    def forward(self, rows: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError


# ---- registries -----------------------------------------------------------------------------

MIXERS: dict[str, Callable[..., Mixer]] = {}
FEED_FORWARDS: dict[str, Callable[..., FeedForward]] = {}
NORMS: dict[str, Callable[..., Norm]] = {}
POSITION_ENCODINGS: dict[str, Callable[..., PositionEncoding]] = {}
EMBEDDINGS: dict[str, Callable[..., Embedding]] = {}
HEADS: dict[str, Callable[..., Head]] = {}
BLOCKS: dict[str, Callable[..., Any]] = {}

_TABLES = {"mixer": MIXERS, "feed_forward": FEED_FORWARDS, "norm": NORMS,
           "position_encoding": POSITION_ENCODINGS, "embedding": EMBEDDINGS, "head": HEADS, "block": BLOCKS}


def register(family: str, name: str) -> Callable:
    """`@register("mixer", "my_mixer")` above a class (or, for blocks, a function)."""
    table = _TABLES[family]

    def deco(obj):
        table[name] = obj
        return obj

    return deco


@dataclass(frozen=True)
class PartSpec:
    """A part chosen by name with its constructor arguments (sizes and constants only)."""

    kind: str
    args: dict[str, Any] = field(default_factory=dict)


def make(family: str, spec: PartSpec):
    table = _TABLES[family]
    if spec.kind not in table:
        raise KeyError(f"no {family} named {spec.kind!r}; registered: {sorted(table)}")
    return table[spec.kind](**spec.args)

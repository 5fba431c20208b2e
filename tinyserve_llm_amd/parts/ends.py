"""The two ends of a model: the table that turns token ids into hidden rows, and the projection
that turns the final rows into logits (tinyserve_llm/model/llama.py:262-268,293-304: an embedding
module, and a head that is the embedding's weight when the checkpoint ties them). Another
architecture that scales its embeddings or caps its logits registers parts of its own under
"embedding" and "head"."""

from __future__ import annotations

import torch

from tinyserve_llm_amd.ops import hip
from tinyserve_llm_amd.parts.base import Embedding, Head, ParamSpec, StepContext, register
from tinyserve_llm_amd.parts.linear import linear, streaming_copy


@register("embedding", "table")
class TableEmbedding(Embedding):
    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int, init: tuple[float, float] = (0.0, 0.02)) -> None:
        self.vocab_size, self.hidden_size, self.init = vocab_size, hidden_size, tuple(init)
        self.weight: torch.Tensor | None = None

    def param_specs(self) -> dict[str, ParamSpec]:
        return {"weight": ParamSpec((self.vocab_size, self.hidden_size), init=self.init)}

    def table(self) -> torch.Tensor | None:
        return self.weight

    def forward(self, ctx: StepContext) -> torch.Tensor:
        return hip.embedding(self.weight, ctx.token_ids)      # (ids are checked against the vocabulary on the host)


@register("head", "projection")
class ProjectionHead(Head):
    """float32 logits = rows · Wᵀ with W [vocab, hidden], its own or the embedding's."""

    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int, tied: bool = False, init: tuple[float, float] = (0.0, 0.02)) -> None:
        self.vocab_size, self.hidden_size, self.tied, self.init = vocab_size, hidden_size, tied, tuple(init)
        self.weight: torch.Tensor | None = None
        self.weight_packed = None                # `streaming_copy` of the weight, if the model keeps them

    def param_specs(self) -> dict[str, ParamSpec]:
        return {} if self.tied else {"weight": ParamSpec((self.vocab_size, self.hidden_size), init=self.init)}

    def tie(self, table: torch.Tensor) -> None:
        if table is None or tuple(table.shape) != (self.vocab_size, self.hidden_size):
            raise ValueError(f"a tied head needs the embedding's [{self.vocab_size}, {self.hidden_size}] table")
        self.weight = table

    def keep_streaming_copies(self) -> int:
        # (a step reads the whole vocabulary matrix once whatever its size: at the 1B sizes a fifth of a decode step's bytes)
        self.weight_packed = streaming_copy(self.weight)
        return 0 if self.weight_packed is None else self.weight_packed.nbytes()

    def forward(self, rows: torch.Tensor) -> torch.Tensor:
        return linear(rows, self.weight, out_dtype=torch.float32, packed=self.weight_packed)

"""A request's sampling options and the scheduler's record of one sequence
(tinyserve_llm/scheduler/sequence.py:8-56)."""

from __future__ import annotations

from dataclasses import dataclass, field
from enum import Enum, auto
from typing import Literal


@dataclass(frozen=True)
class SamplingParams:
    max_tokens: int = 256
    temperature: float = 1.0     # 0 = greedy
    n: int = 1                   # parallel samples of one prompt
    ignore_eos: bool = False


class SequenceStatus(Enum):
    WAITING = auto()
    RUNNING = auto()
    FINISHED = auto()


@dataclass
class Sequence:
    seq_id: int
    request_id: int                      # shared by the n samples of a request
    prompt_token_ids: tuple[int, ...]
    params: SamplingParams
    arrival_time: float                  # kept through preemptions
    status: SequenceStatus = SequenceStatus.WAITING
    output_token_ids: list[int] = field(default_factory=list)
    sample_index: int = 0                # which of the request's n samples this is
    admission_hit: float = 0.0           # cache hit at the last admission; ranks the sequence while it runs
    num_preemptions: int = 0
    first_token_time: float | None = None
    finish_time: float | None = None
    finish_reason: Literal["eos", "length"] | None = None
    # prompt feeding: what the current admission has to put into the cache, and how far it got
    prefill_target: int = 0              # number of leading tokens of all_token_ids to be cached before decoding
    num_computed: int = 0                # tokens whose keys/values are committed in the cache
    in_step: bool = False                # scheduled in the step that is being built or run

    @property
    def pending_token(self) -> int:
        """The newest sampled token: it has no keys/values yet, the next decode step feeds it."""
        return self.output_token_ids[-1]

    @property
    def all_token_ids(self) -> list[int]:
        return [*self.prompt_token_ids, *self.output_token_ids]

    @property
    def num_tokens(self) -> int:
        return len(self.prompt_token_ids) + len(self.output_token_ids)

    @property
    def in_prefill(self) -> bool:
        return self.num_computed < self.prefill_target

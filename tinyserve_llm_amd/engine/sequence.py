"""What a request asks of the sampler, and the scheduler's record of one sequence of tokens
(tinyserve_llm/scheduler/sequence.py:8-56 keeps the same public fields; the portion counters,
the step flag and the methods are this engine's)."""

from __future__ import annotations

from dataclasses import dataclass, field
from enum import Enum, auto
from typing import Literal


@dataclass(frozen=True)
class SamplingParams:
    max_tokens: int = 256
    temperature: float = 1.0     # 0: always the most likely token
    n: int = 1                   # how many continuations of the prompt are drawn side by side
    ignore_eos: bool = False


class SequenceStatus(Enum):
    WAITING = auto()
    RUNNING = auto()
    FINISHED = auto()


@dataclass
class Sequence:
    seq_id: int
    request_id: int                      # the same for all n continuations of one prompt
    prompt_token_ids: tuple[int, ...]
    params: SamplingParams
    arrival_time: float                  # of the request; a preemption does not reset it
    status: SequenceStatus = SequenceStatus.WAITING
    output_token_ids: list[int] = field(default_factory=list)
    sample_index: int = 0                # 0 .. n-1: which continuation of its request (names its draws' noise)
    admission_hit: float = 0.0           # share of it found in the cache when it was last admitted: its rank while running
    num_preemptions: int = 0
    first_token_time: float | None = None
    finish_time: float | None = None
    finish_reason: Literal["eos", "length"] | None = None
    # feeding: an admission has to bring the first `prefill_target` tokens into the cache, in one
    # portion or several, before the sequence decodes; `num_computed` of them are in so far
    prefill_target: int = 0
    num_computed: int = 0                # tokens whose keys/values are committed in the cache
    in_step: bool = False                # part of the step that is being built or is running

    @property
    def pending_token(self) -> int:
        """The newest drawn token: not in the cache yet, the next decode step feeds it."""
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

    def awaits_first_token(self) -> bool:
        """True for the one sequence of a request with n > 1 before its prompt has given a token:
        the other n - 1 are split off it then."""
        return self.params.n > 1 and not self.output_token_ids

    def why_it_ends(self, eos_token_id: int) -> Literal["eos", "length"] | None:
        """Whether the newest token is the sequence's last, and why."""
        if not self.params.ignore_eos and self.output_token_ids[-1] == eos_token_id:
            return "eos"
        return "length" if len(self.output_token_ids) >= self.params.max_tokens else None

    def continuation(self, seq_id: int, sample_index: int) -> "Sequence":
        """Another continuation of the same prompt, to be split off before the first token: it
        starts where this one stands (same portion counters, same rank), with no outputs."""
        if self.output_token_ids:
            raise AssertionError("continuations part before the first token")
        return Sequence(seq_id, self.request_id, self.prompt_token_ids, self.params, self.arrival_time,
                        status=self.status, sample_index=sample_index, admission_hit=self.admission_hit,
                        prefill_target=self.prefill_target, num_computed=self.num_computed)

    def start_running(self, hit: float, target: int, computed: int) -> None:
        """Admitted: `computed` of its first `target` tokens were found in the cache."""
        self.status, self.admission_hit = SequenceStatus.RUNNING, hit
        self.prefill_target, self.num_computed, self.in_step = target, computed, True

    def back_to_waiting(self) -> None:
        """Preempted: nothing of it is in the cache any more; outputs and arrival time stay."""
        self.status = SequenceStatus.WAITING
        self.num_preemptions += 1
        self.prefill_target = self.num_computed = 0

    def finish(self, reason: Literal["eos", "length"], now: float) -> None:
        self.status, self.finish_reason, self.finish_time = SequenceStatus.FINISHED, reason, now

"""The scheduler: admits requests by cache hit and age, cuts prompts into portions under a token
budget, decodes, forks parallel samples, finishes and frees, and preempts when pages run out
(tinyserve_llm/scheduler/scheduler.py:12-267). It is host code and talks to the cache manager only.

Beyond the reference: a prompt need not fit one step. An admission feeds the first portion of the
uncached tokens (as much as the step's budget and `max_prefill_chunk` allow); a sequence that is
still inside its prompt feeds the next portion each step, after the decodes and before new
admissions; only the final portion yields a token.

A decode step can be closed in two halves, `commit_decodes` (all that does not depend on the drawn
tokens) and `deliver_tokens` (all that does), with a `schedule` for the next step in between: the
engine schedules and packs step n+1 while the device still runs step n. Between the halves a
sequence's newest output is the placeholder `PENDING`; the next step feeds the placeholder, and
delivery puts the token in its place (in the sequence, in the scheduled entry and in the cache
manager's record of the slot).

When pages run out: a running sequence that cannot get the page it needs makes the lowest-ranked
sequences not yet scheduled in this step give up theirs (preemption: pages released, which keeps
them in the prefix cache while nobody else needs them; the sequence returns to the waiting queue
with its outputs and its arrival time); if none is left it gives up its own and this kind of
scheduling stops for the step.
"""

from __future__ import annotations

import itertools
import math
import operator
from collections import Counter
from dataclasses import dataclass
from typing import Literal, NamedTuple

from tinyserve_llm_amd.cache.manager import AdmissionCost, KVCacheManager
from tinyserve_llm_amd.engine.sequence import SamplingParams, Sequence, SequenceStatus


@dataclass(frozen=True)
class SchedulerConfig:
    max_model_len: int = 4096
    max_num_seqs: int = 512
    max_num_batched_tokens: int = 16384
    eos_token_id: int = -1
    wait_weight: float = 0.1            # score = hit + wait_weight * seconds waited
    hit_mode: Literal["absolute", "ratio"] = "absolute"
    max_skip_wait: float = 5.0          # a misfit that waited this long stops admission behind it
    watermark: float = 0.01             # fraction of pages kept free at admission
    step_mode: Literal["mixed", "prefill_first"] = "mixed"
    max_prefill_chunk: int = 0          # most prompt tokens of one sequence per step; 0 = the budget

    def __post_init__(self) -> None:
        # every running sequence decodes first; one more token must remain for a prompt portion
        assert self.max_num_batched_tokens >= self.max_num_seqs + 1, \
            "the token budget could be used up by decodes alone"
        assert self.max_prefill_chunk >= 0


@dataclass
class SchedulerStats:
    admissions: int = 0
    readmissions: int = 0
    preemptions: int = 0
    cached_tokens: int = 0
    prefill_tokens: int = 0
    decode_tokens: int = 0
    num_waiting: int = 0
    num_running: int = 0


PENDING = -1      # stands in for a token that the device has drawn and the host has not read yet


class ScheduledSeq(NamedTuple):
    seq: Sequence
    token_ids: list[int]      # fed this step, at positions start .. start + len - 1
    num_samples: int = 1      # 0 for a portion that does not end the prompt; n on a group's first token
    start: int = 0


_START = operator.attrgetter("start")


class _Offer(NamedTuple):
    """The terms of one admission: the sequence's tokens, how many of the uncached ones the step
    would feed, the pages that takes in every page space, the share of the sequence found in the
    cache, and the samples it will split off at its first token."""
    tokens: list[int]
    feed: int
    per_space: list[int]
    hit: float
    forks: int


class RequestOutput(NamedTuple):
    request_id: int
    sequences: list[Sequence]


class Scheduler:
    def __init__(self, config: SchedulerConfig, kv: KVCacheManager) -> None:
        self.config = config
        self.kv = kv
        self.waiting: list[Sequence] = []
        self.running: list[Sequence] = []
        self.groups: dict[int, list[Sequence]] = {}
        self.watermark_blocks = math.ceil(config.watermark * kv.num_blocks)
        self._seq_ids = itertools.count()
        self._request_ids = itertools.count()
        self.tally: Counter[str] = Counter()       # the running totals of `SchedulerStats`, by field name

    def has_unfinished(self) -> bool:
        return bool(self.waiting or self.running)

    # ---- arrival ----------------------------------------------------------------------------
    def add_request(self, prompt_token_ids: list[int], params: SamplingParams, arrival_time: float) -> int:
        """Queues a request; refuses one that could never run (scheduler.py:67-87)."""
        assert prompt_token_ids and params.max_tokens >= 1 and params.n >= 1
        longest = len(prompt_token_ids) + params.max_tokens
        if longest > self.config.max_model_len:
            raise ValueError(f"prompt + max_tokens = {longest} exceeds max_model_len")
        # one sequence at full length, a page per further sample, the watermark, and one page for
        # the source of a partial-page copy that must exist beside its destination
        worst = -(-longest // self.kv.block_size) + (params.n - 1) + self.watermark_blocks + 1
        if worst > self.kv.num_blocks:
            raise ValueError(f"needs up to {worst} blocks; the KV cache has {self.kv.num_blocks}")
        if params.n > self.config.max_num_seqs:
            raise ValueError(f"n = {params.n} samples exceed max_num_seqs")
        request_id = next(self._request_ids)
        seq = Sequence(next(self._seq_ids), request_id, tuple(prompt_token_ids), params, arrival_time)
        self.groups[request_id] = [seq]
        self.waiting.append(seq)
        return request_id

    # ---- ranking ----------------------------------------------------------------------------
    def _hit(self, num_tokens: int, cost: AdmissionCost) -> float:
        cached = num_tokens - cost.prefill_tokens
        return cached / (self.config.max_model_len if self.config.hit_mode == "absolute" else num_tokens)

    def _score(self, hit: float, seq: Sequence, now: float) -> float:
        return hit + self.config.wait_weight * (now - seq.arrival_time)

    def _ranked_waiting(self, now: float) -> list[tuple[Sequence, float]]:
        ranked = []
        for seq in self.waiting:
            if seq.output_token_ids and seq.output_token_ids[-1] == PENDING:
                continue                           # preempted with a token under way: it waits for the token
            tokens = seq.all_token_ids
            hit = self._hit(len(tokens), self.kv.calculate_admission_cost(tokens))
            ranked.append((self._score(hit, seq, now), seq))
        ranked.sort(key=lambda r: r[0], reverse=True)
        return [(seq, score) for score, seq in ranked]

    def _chunk(self, left: int, budget: int) -> int:
        cap = self.config.max_prefill_chunk or budget
        return max(0, min(left, budget, cap))

    # ---- one step ---------------------------------------------------------------------------
    def schedule(self, now: float) -> list[ScheduledSeq]:
        budget = self.config.max_num_batched_tokens
        if self.config.step_mode == "prefill_first":
            prompts = self._schedule_running(now, budget, want_prefill=True)
            prompts += self._admit(now, budget - sum(len(s.token_ids) for s in prompts))
            return prompts or self._longest_first(self._schedule_running(now, budget, want_prefill=False))
        decodes = self._longest_first(self._schedule_running(now, budget, want_prefill=False))
        budget -= len(decodes)
        portions = self._schedule_running(now, budget, want_prefill=True)
        budget -= sum(len(s.token_ids) for s in portions)
        return decodes + portions + self._admit(now, budget)

    @staticmethod
    def _longest_first(decodes: list[ScheduledSeq]) -> list[ScheduledSeq]:
        """The step's decoding requests in the order of their context lengths, longest first. Who
        is in the step is decided; the order inside it is free, and the attention kernel's
        workgroups start in this order: with neighbours of similar length, the longest first, 64
        requests of 768 to 4,352 tokens take it 133 µs a layer instead of 167."""
        decodes.sort(key=_START, reverse=True)
        return decodes

    def _schedule_running(self, now: float, budget: int, want_prefill: bool) -> list[ScheduledSeq]:
        """Feeds running sequences of one kind (inside their prompt, or decoding), best score
        first. Victims of a page shortage are the lowest-ranked sequences of either kind that
        this step has not scheduled."""
        mine = [s for s in self.running if s.in_prefill == want_prefill and not s.in_step]
        if want_prefill or budget < len(mine) or not self.kv.fits([len(mine)] * len(self.kv.spaces)):
            mine.sort(key=lambda s: self._score(s.admission_hit, s, now))       # lowest first
        # (decoding sequences that all fit, in tokens and in pages, a page each at most, need no ranking:
        # all of them run, and the step lays them out by context length anyway)
        scheduled: list[ScheduledSeq] = []
        gone: set[int] = set()
        while mine:
            seq = mine.pop()
            if want_prefill:
                n = self._chunk(seq.prefill_target - seq.num_computed, budget)
                if n == 0:
                    continue                       # no budget left for it this step; it keeps its pages
                tokens = seq.all_token_ids[seq.num_computed:seq.num_computed + n]
            else:
                if budget <= 0:
                    continue
                if seq.output_token_ids[-1] == PENDING and len(seq.output_token_ids) >= seq.params.max_tokens:
                    continue                       # the token under way is its last one
                tokens = [seq.pending_token]
            one = not want_prefill       # a decoded token: asked for and reserved in one call
            fits = self.kv.try_append_one(seq.seq_id, tokens[0]) if one else self.kv.can_append(seq.seq_id, len(tokens))
            while not fits:
                victim = self._lowest_unscheduled(now, exclude=seq, gone=gone)
                if victim is None:
                    break
                self._send_back(victim)
                gone.add(victim.seq_id)
                if victim in mine:
                    mine.remove(victim)
                fits = self.kv.try_append_one(seq.seq_id, tokens[0]) if one else self.kv.can_append(seq.seq_id, len(tokens))
            if not fits:
                self._send_back(seq)
                gone.add(seq.seq_id)
                break
            if not one:
                self.kv.append_slots(seq.seq_id, tokens, checked=True)
            final = seq.num_computed + len(tokens) >= seq.prefill_target
            samples = 1
            if want_prefill:
                samples = 0 if not final else (seq.params.n if seq.awaits_first_token() else 1)
                self.tally["prefill_tokens"] += len(tokens)
            else:
                self.tally["decode_tokens"] += 1
            seq.in_step = True
            scheduled.append(ScheduledSeq(seq, tokens, samples, seq.num_computed))
            budget -= len(tokens)
        return scheduled

    def _lowest_unscheduled(self, now: float, exclude: Sequence, gone: set[int]) -> Sequence | None:
        pool = [s for s in self.running if s is not exclude and s.seq_id not in gone
                and not s.in_step]
        return min(pool, key=lambda s: self._score(s.admission_hit, s, now), default=None)

    def _send_back(self, seq: Sequence) -> None:
        """Preemption (scheduler.py:152-158): the sequence leaves the running list for the end of the
        waiting queue, keeping its outputs and its place in time; its pages go back to the manager,
        where they stay findable by prefix while nobody needs them."""
        self.running.remove(seq)
        self.kv.release(seq.seq_id)
        seq.back_to_waiting()
        self.waiting.append(seq)
        self.tally["preemptions"] += 1

    def _owed_forks(self) -> int:
        """Sequences that running requests will still split off when their prompts end."""
        return sum(s.params.n - 1 for s in self.running if s.awaits_first_token())

    def _offer(self, seq: Sequence, budget: int) -> "_Offer":
        """What admitting `seq` now would feed and take, priced against the cache as it is at this
        moment (an admission made a moment ago may have evicted pages an older price counted on)."""
        tokens = seq.all_token_ids
        whole = self.kv.calculate_admission_cost(tokens)
        feed = self._chunk(whole.prefill_tokens, budget)
        return _Offer(tokens, feed, self.kv.calculate_admission_cost(tokens, feed).per_space,
                      self._hit(len(tokens), whole), seq.params.n - 1 if seq.awaits_first_token() else 0)

    def _room_for(self, offer: "_Offer", owed: int) -> bool:
        """Seats: the sequence and every sample it or an earlier admission still owes. Pages: its own,
        one per owed sample (the copy of a shared last page), and the watermark."""
        seats = len(self.running) + owed + offer.forks + 1
        return (offer.feed >= 1 and seats <= self.config.max_num_seqs
                and self.kv.fits(offer.per_space, owed + offer.forks + self.watermark_blocks))

    def _seat(self, seq: Sequence, offer: "_Offer") -> ScheduledSeq:
        """Makes the admission: pages reserved for the first portion, the books updated."""
        took = self.kv.allocate(seq.seq_id, offer.tokens, offer.feed)
        assert took is not None, "the price was taken a moment ago"
        cached = self.kv.num_cached_tokens(seq.seq_id)
        fed = offer.tokens[cached:cached + offer.feed]
        self.tally["readmissions" if seq.num_preemptions else "admissions"] += 1
        self.tally["cached_tokens"] += cached
        self.tally["prefill_tokens"] += len(fed)
        seq.start_running(offer.hit, target=len(offer.tokens), computed=cached)
        self.running.append(seq)
        ends_prompt = cached + len(fed) >= len(offer.tokens)
        return ScheduledSeq(seq, fed, (offer.forks + 1) if ends_prompt else 0, cached)

    def _admit(self, now: float, budget: int) -> list[ScheduledSeq]:
        """New admissions of a step (the policy of scheduler.py:160-204, over portions): waiting
        sequences are offered a seat in the order of their scores; one that has no room is passed
        over, except that one which has waited `max_skip_wait` ends the round, so that what frees up
        next goes to it and not to smaller requests behind it."""
        seated: list[ScheduledSeq] = []
        owed = self._owed_forks()
        if not self.waiting or len(self.running) + owed >= self.config.max_num_seqs:
            return seated                        # nobody to admit or no seat: no ranking needed
        for seq, _ in (self._ranked_waiting(now) if budget > 0 else ()):
            offer = self._offer(seq, budget)
            if not self._room_for(offer, owed):
                if now - seq.arrival_time < self.config.max_skip_wait:
                    continue
                break
            entry = self._seat(seq, offer)
            seated.append(entry)
            owed += offer.forks
            budget -= len(entry.token_ids)
            if budget <= 0:
                break
        if seated:
            self.waiting = [s for s in self.waiting if s.status is SequenceStatus.WAITING]
        return seated

    # ---- after the model ran ----------------------------------------------------------------
    def _split_off(self, first: Sequence, how_many: int) -> list[Sequence]:
        """The sequences that take the `how_many` tokens drawn from a prompt's last position: the
        one that was fed, and for n > 1 its new siblings, which share all its pages."""
        family = [first]
        for index in range(1, how_many):
            sibling = first.continuation(next(self._seq_ids), index)
            self.kv.fork(first.seq_id, sibling.seq_id)
            self.running.append(sibling)
            self.groups[first.request_id].append(sibling)
            family.append(sibling)
        return family

    def _retire(self, ended: list[Sequence]) -> list[RequestOutput]:
        """Takes ended sequences off the running list; a request whose sequences have all ended is
        handed out, in the order in which the requests' last sequences ended."""
        if not ended:
            return []
        gone = {s.seq_id for s in ended}
        self.running = [s for s in self.running if s.seq_id not in gone]
        complete = []
        for seq in ended:
            family = self.groups.get(seq.request_id)
            if family is not None and all(s.status is SequenceStatus.FINISHED for s in family):
                complete.append(RequestOutput(seq.request_id, self.groups.pop(seq.request_id)))
        return complete

    def postprocess(self, scheduled: list[ScheduledSeq], sampled: list[list[int]], now: float) -> list[RequestOutput]:
        """Closes a step in one piece: every entry's slots are committed; where tokens were drawn, the
        sequence (for n > 1: it and the siblings split off it now) takes them, and what ends with
        its token gives its pages back (the reference's counterpart is scheduler.py:236-263)."""
        ended: list[Sequence] = []
        for (seq, token_ids, num_samples, _), tokens in zip(scheduled, sampled, strict=True):
            assert len(tokens) == num_samples
            seq.in_step = False
            self.kv.commit(seq.seq_id, len(token_ids))
            seq.num_computed += len(token_ids)
            if not tokens:
                continue                                   # a portion that does not end its prompt
            for taker, token in zip(self._split_off(seq, num_samples), tokens):
                taker.output_token_ids.append(token)
                taker.prefill_target = taker.num_computed  # from here on it decodes
                if taker.first_token_time is None:
                    taker.first_token_time = now
                reason = taker.why_it_ends(self.config.eos_token_id)
                if reason is not None:
                    self.kv.release(taker.seq_id)
                    taker.finish(reason, now)
                    ended.append(taker)
        return self._retire(ended)

    # ---- the same for decode steps, in two halves -------------------------------------------------
    @staticmethod
    def decodes_only(scheduled: list[ScheduledSeq]) -> bool:
        """Whether every entry of the step feeds one decoded token and draws one."""
        return all(len(b.token_ids) == 1 and b.num_samples == 1 and b.seq.output_token_ids for b in scheduled)

    def commit_decodes(self, scheduled: list[ScheduledSeq]) -> None:
        """First half of `postprocess` for a step of decodes only: what does not depend on the
        tokens drawn. Each sequence's newest output is `PENDING` until `deliver_tokens`."""
        for seq, token_ids, num_samples, _ in scheduled:
            assert len(token_ids) == 1 and num_samples == 1 and seq.output_token_ids
            seq.in_step = False
            self.kv.commit(seq.seq_id, 1)
            seq.num_computed += 1
            seq.prefill_target = seq.num_computed
            seq.output_token_ids.append(PENDING)

    def deliver_tokens(self, scheduled: list[ScheduledSeq], sampled: list[list[int]], now: float,
                       ahead: list[ScheduledSeq] | None = None) -> tuple[list[RequestOutput], list[ScheduledSeq]]:
        """Second half: the drawn tokens take the placeholders' place, what finished is released.
        `ahead` is the step scheduled in between: its entries that feed a placeholder get the token,
        entries of sequences that turn out finished are dropped. Returns the finished requests and
        what is left of `ahead`."""
        ended: list[Sequence] = []
        fed_ahead = {b.seq.seq_id: b for b in ahead or ()}
        for (seq, _, _, _), tokens in zip(scheduled, sampled, strict=True):
            assert len(tokens) == 1 and seq.output_token_ids[-1] == PENDING
            token = tokens[0]
            seq.output_token_ids[-1] = token
            entry = fed_ahead.get(seq.seq_id)
            reason = seq.why_it_ends(self.config.eos_token_id)
            if reason is None:
                if entry is not None:
                    assert entry.token_ids == [PENDING] and entry.start == seq.num_computed
                    entry.token_ids[0] = token
                    self.kv.set_token(seq.seq_id, entry.start, token)
                continue
            if seq.status is SequenceStatus.RUNNING:
                if entry is not None:              # scheduled again before anyone knew: the slot goes back
                    self.kv.commit(seq.seq_id, 0)
                    seq.in_step = False
                    del fed_ahead[seq.seq_id]
                self.kv.release(seq.seq_id)
            else:                                  # preempted in between: its pages went back then
                self.waiting = [s for s in self.waiting if s.seq_id != seq.seq_id]
            seq.finish(reason, now)
            ended.append(seq)
        return self._retire(ended), [b for b in ahead or () if b.seq.seq_id in fed_ahead]

    def stats(self) -> SchedulerStats:
        """The totals so far and the lengths of the two queues as they are now."""
        return SchedulerStats(num_waiting=len(self.waiting), num_running=len(self.running), **self.tally)

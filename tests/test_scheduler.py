"""The scheduler's decisions on the CPU, with a stand-in model whose next token is a function of
the history it reads back from the cache slots: a wrong feed, a wrong position or a lost page
changes what is generated. Fixed cases follow what the reference's tests pin
(tests/test_scheduler.py), cited at each; portions of prompts are this engine's own."""

from __future__ import annotations

import random

import pytest

from tests.test_cache_manager import B, FakeStorage, check_invariants, forward
from tinyserve_llm_amd.cache.manager import KVCacheManager
from tinyserve_llm_amd.engine.scheduler import Scheduler, SchedulerConfig
from tinyserve_llm_amd.engine.sequence import SamplingParams, SequenceStatus

VOCAB, EOS = 8, 1


def model(history, sample):
    """Next token from everything before it (and which sample is drawn); never EOS by itself."""
    return hash((tuple(history), sample)) % VOCAB + 2


def config(**over):
    base = dict(max_model_len=64, max_num_seqs=8, max_num_batched_tokens=72, eos_token_id=EOS, watermark=0.0)
    return SchedulerConfig(**{**base, **over})


def make(pages=32, caching=True, **over):
    return Scheduler(config(**over), KVCacheManager(FakeStorage(pages), caching=caching))


def check_scheduler(s):
    m = s.kv
    check_invariants(m)
    assert {q.seq_id for q in s.running}.isdisjoint(q.seq_id for q in s.waiting)
    assert set(m.seqs) == {q.seq_id for q in s.running}, "exactly the running sequences hold pages"
    assert len(s.running) <= s.config.max_num_seqs
    for q in s.running:
        assert q.status is SequenceStatus.RUNNING and not q.in_step
        st = m.seqs[q.seq_id]
        assert st.committed == q.num_computed
        if q.in_prefill:
            assert st.token_ids == q.all_token_ids[:q.num_computed]
        else:
            assert st.token_ids == q.all_token_ids[:-1], "every token but the pending one is cached"
    for q in s.waiting:
        assert q.status is SequenceStatus.WAITING
    for group in s.groups.values():
        assert len(group) <= group[0].params.n


def run_step(s, now, token_for=model):
    m = s.kv
    batch = s.schedule(now)
    assert sum(len(b.token_ids) for b in batch) <= s.config.max_num_batched_tokens
    assert len({b.seq.seq_id for b in batch}) == len(batch)
    sampled = []
    for seq, fed, num_samples, start in batch:
        st = m.seqs[seq.seq_id]
        assert st.committed == start and st.token_ids[start:] == list(fed), "positions start where the cache ends"
        assert list(fed) == seq.all_token_ids[start:start + len(fed)]
        forward(m, seq.seq_id)
        history = [m.storage.slots[0][st.block_table[p // B]][p % B] for p in range(st.reserved)]
        sampled.append([token_for(history, k) for k in range(num_samples)])
    outputs = s.postprocess(batch, sampled, now)
    check_scheduler(s)
    return batch, outputs


class AheadLoop:
    """The engine's other order of a step: a step of decodes only is closed in two halves, with the
    schedule of the next step in between (the device would still be running then)."""

    def __init__(self, s, token_for=model):
        self.s, self.token_for, self.ahead = s, token_for, None
        self.used_ahead = 0

    def launch(self, batch):
        m = self.s.kv
        sampled = []
        for seq, fed, num_samples, start in batch:
            st = m.seqs[seq.seq_id]
            assert st.committed == start and st.token_ids[start:] == list(fed), "positions start where the cache ends"
            assert list(fed) == seq.all_token_ids[start:start + len(fed)] and -1 not in fed
            forward(m, seq.seq_id)
            history = [m.storage.slots[0][st.block_table[p // B]][p % B] for p in range(st.reserved)]
            sampled.append([self.token_for(history, k) for k in range(num_samples)])
        return sampled

    def step(self, now):
        s = self.s
        batch, self.ahead = (self.ahead, None) if self.ahead else (s.schedule(now), None)
        assert sum(len(b.token_ids) for b in batch) <= s.config.max_num_batched_tokens
        sampled = self.launch(batch)
        if s.decodes_only(batch):
            s.commit_decodes(batch)
            nxt = s.schedule(now + 0.05) if s.has_unfinished() else []
            outputs, nxt = s.deliver_tokens(batch, sampled, now, nxt)
            self.ahead = nxt or None
            self.used_ahead += 1
            held = {b.seq.seq_id for b in nxt}
            if not nxt:
                check_invariants(s.kv)                # it expects no open reservation
            assert set(s.kv.seqs) == {q.seq_id for q in s.running}, "exactly the running sequences hold pages"
            for q in s.running:                       # the same state as after a whole postprocess and a schedule
                st = s.kv.seqs[q.seq_id]
                assert q.in_step == (q.seq_id in held) and st.committed == q.num_computed
                assert -1 not in st.token_ids and -1 not in q.output_token_ids, "no placeholder outlives the delivery"
                assert st.token_ids == q.all_token_ids[:st.reserved]
            for b in nxt:
                assert -1 not in b.token_ids and list(b.token_ids) == b.seq.all_token_ids[b.start:b.start + len(b.token_ids)]
        else:
            outputs = s.postprocess(batch, sampled, now)
            check_scheduler(s)
        return batch, outputs


def unbatched(prompt, params, sample):
    out = [model(prompt, sample)]
    while not ((out[-1] == EOS and not params.ignore_eos) or len(out) == params.max_tokens):
        out.append(model(prompt + out, 0))
    return out


def run_all(s, max_steps=3000):
    done, now = {}, 0.0
    for _ in range(max_steps):
        if not s.has_unfinished():
            return done
        now += 0.1
        for o in run_step(s, now)[1]:
            assert o.request_id not in done
            done[o.request_id] = o
    raise AssertionError("the scheduler stopped making progress")


# ---- configuration and arrival (tests/test_scheduler.py:113-148) ----------------------------------

def test_budget_must_leave_a_token_beside_the_decodes():
    with pytest.raises(AssertionError):
        SchedulerConfig(max_num_seqs=8, max_num_batched_tokens=8)
    SchedulerConfig(max_num_seqs=8, max_num_batched_tokens=9)


def test_requests_that_can_never_run_are_refused():
    s = make(pages=8)
    with pytest.raises(ValueError, match="max_model_len"):
        s.add_request([1] * 60, SamplingParams(max_tokens=5), 0.0)
    with pytest.raises(ValueError, match="blocks"):
        s.add_request([1] * 20, SamplingParams(max_tokens=10), 0.0)      # 8 pages + 1 > 8
    with pytest.raises(ValueError, match="max_num_seqs"):
        make(pages=32).add_request([1, 2], SamplingParams(max_tokens=2, n=9), 0.0)
    assert s.add_request([1] * 20, SamplingParams(max_tokens=8), 0.0) == 0   # 7 + 1 pages


# ---- portions ----------------------------------------------------------------------------------------

def test_a_long_prompt_is_cut_under_the_budget_and_only_its_end_samples():
    s = make(max_num_batched_tokens=20, max_num_seqs=4)
    s.add_request(list(range(2, 52)) , SamplingParams(max_tokens=3, ignore_eos=True), 0.0)
    shapes = []
    while s.has_unfinished():
        batch, _ = run_step(s, 1.0)
        shapes.append([(len(b.token_ids), b.num_samples, b.start) for b in batch])
    assert shapes[:3] == [[(20, 0, 0)], [(20, 0, 20)], [(10, 1, 40)]]
    assert shapes[3:] == [[(1, 1, 50)], [(1, 1, 51)]]
    st = s.stats()
    assert (st.prefill_tokens, st.decode_tokens, st.admissions) == (50, 2, 1)


def test_decodes_go_first_and_portions_share_what_is_left():
    s = make(max_num_batched_tokens=12, max_num_seqs=4, max_prefill_chunk=6)
    s.add_request([2, 3, 4], SamplingParams(max_tokens=20, ignore_eos=True), 0.0)
    run_step(s, 0.1)
    s.add_request(list(range(2, 22)) * 1, SamplingParams(max_tokens=2, ignore_eos=True), 0.2)
    s.add_request(list(range(3, 13)), SamplingParams(max_tokens=2, ignore_eos=True), 0.3)
    batch, _ = run_step(s, 0.4)
    # one decode, then 6 tokens of the older prompt (chunk cap), then what is left of the budget
    assert [(len(b.token_ids), b.num_samples) for b in batch] == [(1, 1), (6, 0), (5, 0)]
    batch, _ = run_step(s, 0.5)
    assert [(len(b.token_ids), b.num_samples) for b in batch] == [(1, 1), (6, 0), (5, 1)]


def test_a_steps_decodes_come_longest_context_first():
    """Who decodes in a step is a matter of rank; inside the step the decoding requests are laid
    out by the length of their contexts, which is the order the attention kernel starts them in."""
    s = make(pages=64, max_num_batched_tokens=72, max_num_seqs=8)
    for n, at in ((5, 0.0), (23, 0.1), (2, 0.2), (14, 0.3)):
        s.add_request(list(range(2, 2 + n)), SamplingParams(max_tokens=6, ignore_eos=True), at)
    run_step(s, 0.4)
    for now in (0.5, 0.6):
        batch, _ = run_step(s, now)
        assert all(len(b.token_ids) == 1 for b in batch) and len(batch) == 4
        assert [b.start for b in batch] == sorted((b.start for b in batch), reverse=True)
        assert [len(b.seq.prompt_token_ids) for b in batch] == [23, 14, 5, 2]


def test_portions_and_whole_prompts_generate_the_same():
    prompts = [[2 + (i * 7 + j) % 6 for j in range(n)] for i, n in enumerate((30, 3, 17, 45, 9))]
    params = SamplingParams(max_tokens=6, ignore_eos=True)
    outs = []
    for over in (dict(), dict(max_num_batched_tokens=9), dict(max_prefill_chunk=4), dict(step_mode="prefill_first", max_prefill_chunk=7)):
        s = make(**over)
        ids = [s.add_request(p, params, 0.0) for p in prompts]
        done = run_all(s)
        outs.append([done[i].sequences[0].output_token_ids for i in ids])
        assert s.kv.stats().blocks_in_use == 0
    assert all(o == outs[0] for o in outs)
    assert outs[0] == [unbatched(p, params, 0) for p in prompts]


# ---- ranking (tests/test_scheduler.py:204-251) ---------------------------------------------------------

def test_a_cached_prompt_is_admitted_before_a_cold_one_and_waiting_outranks_a_hit():
    s = make(max_num_batched_tokens=30, max_num_seqs=2)
    warm = list(range(2, 22))
    s.add_request(warm, SamplingParams(max_tokens=1), 0.0)
    run_all(s)
    cold_id = s.add_request([7] * 20, SamplingParams(max_tokens=1), 10.0)
    hot_id = s.add_request(warm + [5], SamplingParams(max_tokens=1), 10.0)
    batch = s.schedule(10.0)
    assert [b.seq.request_id for b in batch] == [hot_id, cold_id] and len(batch[0].token_ids) == 1
    s.postprocess(batch, [[3], [3]], 10.0)
    # a cold request that has waited long enough outranks a fresh fully cached one
    cold_id = s.add_request([6] * 20, SamplingParams(max_tokens=1), 20.0)
    hot_id = s.add_request(warm + [5], SamplingParams(max_tokens=1), 29.0)
    batch = s.schedule(29.0)
    assert [b.seq.request_id for b in batch] == [cold_id, hot_id]


def test_hit_modes():
    for mode, want in (("absolute", 20 / 64), ("ratio", 20 / 21)):
        s = make(hit_mode=mode)
        warm = list(range(2, 22))
        s.add_request(warm, SamplingParams(max_tokens=1), 0.0)
        run_all(s)
        s.add_request(warm + [5], SamplingParams(max_tokens=1), 1.0)
        batch = s.schedule(1.0)
        assert batch[0].seq.admission_hit == pytest.approx(want)


def test_a_misfit_is_skipped_until_it_has_waited_long_enough():
    s = make(pages=12, max_skip_wait=5.0)
    s.add_request([2] * 30, SamplingParams(max_tokens=10, ignore_eos=True), 0.0)
    run_step(s, 0.0)                                                       # holds 8 of 12 pages
    big = s.add_request([3] * 30, SamplingParams(max_tokens=2), 1.0)       # needs 8: does not fit
    small = s.add_request([4] * 5, SamplingParams(max_tokens=2), 2.0)
    batch, _ = run_step(s, 3.0)
    assert small in [b.seq.request_id for b in batch] and big not in [b.seq.request_id for b in batch]
    tiny = s.add_request([5] * 3, SamplingParams(max_tokens=2), 6.5)
    batch, _ = run_step(s, 7.0)                                            # big has waited 6 s: nothing passes it
    assert tiny not in [b.seq.request_id for b in batch]


# ---- caps (tests/test_scheduler.py:262-289) ----------------------------------------------------------------

def test_sequence_cap_counts_the_forks_a_group_still_owes():
    s = make(max_num_seqs=4, max_num_batched_tokens=5)
    a = s.add_request([2] * 9, SamplingParams(max_tokens=3, n=3, ignore_eos=True), 0.0)
    b = s.add_request([3] * 2, SamplingParams(max_tokens=3, n=2, ignore_eos=True), 0.1)
    batch, _ = run_step(s, 1.0)
    # a is admitted (1 running + 2 owed = 3); b would make 5 > 4
    assert [x.seq.request_id for x in batch] == [a] and len(s.waiting) == 1
    batch, _ = run_step(s, 1.1)
    assert [x.num_samples for x in batch] == [3] and len(s.running) == 3
    done = run_all(s)
    assert len(done[a].sequences) == 3 and len(done[b].sequences) == 2


def test_watermark_holds_pages_back_at_admission_only():
    s = make(pages=12, watermark=0.2, max_skip_wait=100.0)
    assert s.watermark_blocks == 3
    s.add_request([2] * 24, SamplingParams(max_tokens=8, ignore_eos=True), 0.0)   # 6 pages now
    s.add_request([3] * 13, SamplingParams(max_tokens=2, ignore_eos=True), 0.0)   # 4 more: 12 - 6 - 3 < 4
    batch, _ = run_step(s, 0.1)
    assert len(batch) == 1 and len(s.waiting) == 1
    for _ in range(8):                                                             # decoding dips into the watermark
        if s.running:
            run_step(s, 0.2)
    assert s.stats().preemptions == 0


# ---- pages run out (tests/test_scheduler.py:316-345) -----------------------------------------------------

def test_the_lowest_ranked_running_sequence_is_preempted():
    s = make(pages=6, max_skip_wait=100.0)
    old = s.add_request([2] * 11, SamplingParams(max_tokens=8, ignore_eos=True), 0.0)
    new = s.add_request([3] * 11, SamplingParams(max_tokens=8, ignore_eos=True), 5.0)
    run_step(s, 5.0)                               # 3 pages each, 12 slots: the next token needs a 4th page... not yet
    run_step(s, 5.1)                               # token 12 fills the pages
    batch, _ = run_step(s, 5.2)                    # both need a page, none is free: the younger gives up
    assert [b.seq.request_id for b in batch] == [old]
    assert s.stats().preemptions == 1 and [q.request_id for q in s.waiting] == [new]
    assert s.waiting[0].num_preemptions == 1 and s.waiting[0].arrival_time == 5.0


def test_a_lone_sequence_preempts_itself_and_comes_back_through_the_cache():
    s = make(pages=6, max_skip_wait=100.0)
    rid = s.add_request([2 + i % 5 for i in range(12)], SamplingParams(max_tokens=6, ignore_eos=True), 0.0)
    run_step(s, 0.1)
    thief = [s.kv.spaces[0].take() for _ in range(3)]        # pages vanish behind the scheduler's back
    assert s.schedule(0.2) == [] and s.stats().preemptions == 1 and not s.running
    for b in thief:
        s.kv.spaces[0].drop(b)
    batch, _ = run_step(s, 0.3)
    st = s.stats()
    assert (st.admissions, st.readmissions, st.preemptions) == (1, 1, 1)
    assert st.cached_tokens == 12, "the released pages were still in the prefix cache"
    assert [len(b.token_ids) for b in batch] == [1], "only the pending token had to run again"
    done = run_all(s)
    params = SamplingParams(max_tokens=6, ignore_eos=True)
    assert done[rid].sequences[0].output_token_ids == unbatched([2 + i % 5 for i in range(12)], params, 0)


def test_preempted_inside_its_prompt_a_sequence_starts_over():
    s = make(pages=8, max_num_batched_tokens=9, max_num_seqs=2, max_skip_wait=100.0, caching=False)
    first = s.add_request([2] * 14, SamplingParams(max_tokens=12, ignore_eos=True), 0.0)
    late = s.add_request([3] * 20, SamplingParams(max_tokens=2, ignore_eos=True), 1.0)
    done = run_all(s)
    st = s.stats()
    assert st.preemptions >= 1, "the pool is too small for both at full length"
    for rid, prompt, mt in ((first, [2] * 14, 12), (late, [3] * 20, 2)):
        want = unbatched(prompt, SamplingParams(max_tokens=mt, ignore_eos=True), 0)
        assert done[rid].sequences[0].output_token_ids == want
    assert s.kv.stats().blocks_in_use == 0


def test_prefill_first_runs_prompts_before_decodes():
    s = make(step_mode="prefill_first")
    s.add_request([2, 3, 4], SamplingParams(max_tokens=4, ignore_eos=True), 0.0)
    run_step(s, 0.1)
    s.add_request([5, 6], SamplingParams(max_tokens=4, ignore_eos=True), 0.2)
    batch, _ = run_step(s, 0.3)
    assert [len(b.token_ids) for b in batch] == [2], "a step of prompts only"
    batch, _ = run_step(s, 0.4)
    assert sorted(len(b.token_ids) for b in batch) == [1, 1], "then both decode"


def test_finish_reasons_and_group_collection():
    s = make()
    eos_after = {"n": 0}

    def token_for(history, k):
        eos_after["n"] += 1
        return EOS if eos_after["n"] == 3 else model(history, k)

    rid = s.add_request([2, 3], SamplingParams(max_tokens=5), 0.0)
    outs = []
    while s.has_unfinished():
        outs += run_step(s, 1.0, token_for)[1]
    (o,) = outs
    assert o.request_id == rid and o.sequences[0].finish_reason == "eos" and len(o.sequences[0].output_token_ids) == 3
    rid = s.add_request([2, 3], SamplingParams(max_tokens=2, n=2, ignore_eos=True), 2.0)
    done = run_all(s)
    assert [q.finish_reason for q in done[rid].sequences] == ["length", "length"]
    assert [q.sample_index for q in done[rid].sequences] == [0, 1]


def test_stats_snapshot_is_a_copy():
    s = make()
    s.add_request([2, 3], SamplingParams(max_tokens=2), 0.0)
    before = s.stats()
    run_step(s, 0.1)
    assert before.admissions == 0 and s.stats().admissions == 1 and before.num_waiting == 1


# ---- random workloads (tests/test_scheduler.py:382-429) -------------------------------------------------

def eos_model(history, sample):
    """Like `model`, but one draw in six is the end token."""
    h = hash((tuple(history), sample))
    return EOS if h % 6 == 0 else h % VOCAB + 2


def unbatched_with(token_for, prompt, params, sample):
    out = [token_for(prompt, sample)]
    while not ((out[-1] == EOS and not params.ignore_eos) or len(out) == params.max_tokens):
        out.append(token_for(prompt + out, 0))
    return out


@pytest.mark.parametrize("seed", range(20))
@pytest.mark.parametrize("caching", [True, False])
def test_random_workload_with_steps_closed_in_two_halves(seed, caching):
    """The same workloads with decode steps closed in two halves around the next schedule, and a
    model that also ends sequences by itself: what was scheduled ahead for a sequence that turns
    out finished goes back, preempted sequences get their token while they wait."""
    rng = random.Random(1000 + seed)
    over = dict(max_num_seqs=rng.choice([2, 4, 8]), max_skip_wait=rng.choice([0.3, 5.0]),
                max_prefill_chunk=rng.choice([0, 3, 8]), step_mode=rng.choice(["mixed", "mixed", "prefill_first"]))
    over["max_num_batched_tokens"] = rng.choice([over["max_num_seqs"] + 1, 16, 72])
    s = make(pages=rng.choice([18, 24, 40]), caching=caching, **over)
    loop = AheadLoop(s, eos_model)
    stems = [[2 + rng.randrange(6) for _ in range(rng.randrange(1, 25))] for _ in range(3)]
    expected, done, now = {}, {}, 0.0
    arrivals = 14
    for step_no in range(4000):
        if arrivals and (rng.random() < 0.3 or not s.has_unfinished()):
            prompt = rng.choice(stems)[:rng.randrange(1, 25)] + [2 + rng.randrange(6) for _ in range(rng.randrange(0, 6))]
            params = SamplingParams(max_tokens=rng.randrange(1, 12), n=rng.choice([1, 1, 2, 3]),
                                    ignore_eos=rng.random() < 0.5)
            if params.n <= over["max_num_seqs"]:
                try:
                    rid = s.add_request(prompt, params, now)
                    expected[rid] = [unbatched_with(eos_model, prompt, params, k) for k in range(params.n)]
                except ValueError:
                    pass
            arrivals -= 1
        if not s.has_unfinished():
            if not arrivals:
                break
            continue
        now += 0.1
        for o in loop.step(now)[1]:
            assert o.request_id not in done
            done[o.request_id] = [q.output_token_ids for q in o.sequences]
    assert not s.has_unfinished() and loop.ahead is None, "the scheduler stopped making progress"
    assert done == expected
    assert loop.used_ahead > 0
    assert s.kv.stats().blocks_in_use == 0 and not s.kv.seqs
    assert len(s.kv.free_state_slots) == s.kv.storage.num_state_slots


@pytest.mark.parametrize("seed", range(20))
@pytest.mark.parametrize("caching", [True, False])
def test_random_workload_equals_unbatched_generation(seed, caching):
    rng = random.Random(seed)
    over = dict(max_num_seqs=rng.choice([2, 4, 8]), max_skip_wait=rng.choice([0.3, 5.0]),
                max_prefill_chunk=rng.choice([0, 3, 8]), step_mode=rng.choice(["mixed", "mixed", "prefill_first"]))
    over["max_num_batched_tokens"] = rng.choice([over["max_num_seqs"] + 1, 16, 72])
    s = make(pages=rng.choice([18, 24, 40]), caching=caching, **over)
    stems = [[2 + rng.randrange(6) for _ in range(rng.randrange(1, 25))] for _ in range(3)]
    expected, done, now = {}, {}, 0.0
    arrivals = 14
    for step_no in range(4000):
        if arrivals and (rng.random() < 0.3 or not s.has_unfinished()):
            prompt = rng.choice(stems)[:rng.randrange(1, 25)] + [2 + rng.randrange(6) for _ in range(rng.randrange(0, 6))]
            params = SamplingParams(max_tokens=rng.randrange(1, 12), n=rng.choice([1, 1, 2, 3]),
                                    ignore_eos=rng.random() < 0.8)
            if params.n <= over["max_num_seqs"]:
                try:
                    rid = s.add_request(prompt, params, now)
                    expected[rid] = [unbatched(prompt, params, k) for k in range(params.n)]
                except ValueError:
                    pass
            arrivals -= 1
        if not s.has_unfinished():
            if not arrivals:
                break
            continue
        now += 0.1
        for o in run_step(s, now)[1]:
            done[o.request_id] = [q.output_token_ids for q in o.sequences]
    assert not s.has_unfinished(), "the scheduler stopped making progress"
    assert done == expected
    assert s.kv.stats().blocks_in_use == 0 and not s.kv.seqs
    assert len(s.kv.free_state_slots) == s.kv.storage.num_state_slots

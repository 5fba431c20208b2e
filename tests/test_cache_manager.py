"""The cache manager on the CPU with a stand-in for device memory whose slots remember which token's
keys they hold: no page is lost, held twice without a count, or freed twice, under fixed cases and
under random orders of requests. Fixed cases restate what the reference's own tests pin
(tests/test_kvcache_manager.py, page size 4, 12 pages), cited at each test."""

from __future__ import annotations

import random

import pytest

from tinyserve_llm_amd.cache.manager import FREED, KVCacheManager, SpaceSpec
from tinyserve_llm_amd.cache.prefix_index import TOP

B = 4


class FakeStorage:
    """Each slot of each space holds the token id whose keys/values it stores (None = never written)."""

    def __init__(self, pages=12, windows=(0,), state_slots=64, keeps_state=False):
        pages = pages if isinstance(pages, (list, tuple)) else [pages] * len(windows)
        self.page_size = B
        self.spaces = [SpaceSpec(n, w) for n, w in zip(pages, windows)]
        self.num_state_slots = state_slots
        self.keeps_state = keeps_state
        self.slots = [[[None] * B for _ in range(n)] for n in pages]
        self.copies: list[tuple[int, int, int]] = []      # of space 0
        self.state = [None] * state_slots

    def copy_slots(self, space, src, dst, n):
        if space == 0:
            self.copies.append((src, dst, n))
        self.slots[space][dst][:n] = self.slots[space][src][:n]

    def copy_state(self, src, dst):
        self.state[dst] = self.state[src]

    def reset_state(self, slot):
        self.state[slot] = 0


def make(pages=12, caching=True, windows=(0,), keeps_state=False):
    return KVCacheManager(FakeStorage(pages, windows, keeps_state=keeps_state), caching=caching)


def forward(m, seq_id):
    """The model's part: write the slots reserved this step, and fold the tokens into the state."""
    s = m.seqs[seq_id]
    for sp, table in enumerate(s.tables):
        for pos in range(s.committed, s.reserved):
            m.storage.slots[sp][table[pos // B]][pos % B] = s.token_ids[pos]
    m.storage.state[s.state_slot] += sum(s.token_ids[s.committed:s.reserved])


def prefill(m, seq_id, prompt, feed=None):
    assert m.allocate(seq_id, prompt, feed) is not None
    s = m.seqs[seq_id]
    forward(m, seq_id)
    m.commit(seq_id, s.reserved - s.committed)


def step(m, seq_id, tokens, accept=None):
    m.append_slots(seq_id, tokens)
    forward(m, seq_id)
    m.commit(seq_id, len(tokens) if accept is None else accept)


def check_invariants(m):
    """Everything the manager promises between steps (after tests/test_kvcache_manager.py:51-83,
    widened to page spaces, windows and state slots)."""
    for sp, space in enumerate(m.spaces):
        holders = [0] * space.num_pages
        for s in m.seqs.values():
            table = s.tables[sp]
            assert s.reserved == s.committed
            assert len(table) == -(-s.committed // B)
            first_needed = max(0, s.committed - space.window + 1) if space.window else 0
            for pos in range(s.committed):
                page = table[pos // B]
                if page == FREED:
                    assert space.window and (pos // B + 1) * B <= first_needed, "a page still in reach was freed"
                    continue
                assert m.storage.slots[sp][page][pos % B] == s.token_ids[pos], "a slot holds another token's keys"
            if space.window:
                for j, page in enumerate(table):   # pages that the window has passed are given back
                    assert (page == FREED) == ((j + 1) * B <= first_needed)
            for page in table:
                if page != FREED:
                    holders[page] += 1
        assert holders == space.holders, "the counts of holders differ from the tables"
        index = space.index
        unheld = {b for b in range(space.num_pages) if space.holders[b] == 0}
        assert sorted(space.idle) == sorted(b for b in unheld if b not in index), "a page is lost or idle twice"
        assert len(set(space.idle)) == len(space.idle)
        assert space.kept == sum(1 for b in unheld if b in index) and set(space.released_at) == {b for b in unheld if b in index}
        # every kept page that nothing follows stands in the queue under the moment of its release
        queued = set(space._queue)
        for b in space.released_at:
            if index.is_leaf(b):
                assert (space.released_at[b], b) in queued, "a kept page could never be evicted"
        if not m.caching or sp:
            assert len(index) == 0
        for b in index:
            tokens, before = index.tokens(b), index.parent(b)
            assert m.storage.slots[sp][b][:len(tokens)] == list(tokens)
            if len(tokens) < B:
                assert index.is_leaf(b)
            if before != TOP:
                assert before in index and len(index.tokens(before)) == B and not index.is_leaf(before)
                if space.holders[b]:
                    assert space.holders[before], "the page before a held page is held"
            # found again by its own tokens, after the pages before it
            path, at = [], b
            while at != TOP:
                path.append(at)
                at = index.parent(at)
            run = [t for page in reversed(path) for t in index.tokens(page)]
            assert index.lookup(run + [0]).pages == list(reversed(path))
        assert sum(index.is_leaf(b) for b in index) <= len(index)
    if m.caching:
        for s in m.seqs.values():
            for i in range(s.committed // B):
                page = s.block_table[i]
                assert m.index.tokens(page) == tuple(s.token_ids[i * B:(i + 1) * B])
                assert m.index.parent(page) == (s.block_table[i - 1] if i else TOP)
    used = [s.state_slot for s in m.seqs.values()]
    assert len(set(used)) == len(used) and not set(used) & set(m.free_state_slots)
    assert sorted(used + m.free_state_slots) == list(range(m.storage.num_state_slots)), "a state slot is lost"
    if m.storage.keeps_state:
        for s in m.seqs.values():
            assert m.storage.state[s.state_slot] == sum(s.token_ids[:s.committed]), \
                "the state slot does not hold this request's state"


# ---- admission (tests/test_kvcache_manager.py:89-199) ---------------------------------------------

def test_cold_prompt_takes_a_page_per_four_tokens():
    m = make()
    cost = m.calculate_admission_cost(list(range(10)))
    assert (cost.blocks_needed, cost.prefill_tokens) == (3, 10)
    assert list(m.allocate(1, list(range(10)))) == [0, 1, 2]
    assert m.num_cached_tokens(1) == 0


def test_a_fully_cached_prompt_still_runs_its_last_token():
    m = make()
    prefill(m, 1, list(range(8)))
    m.release(1)
    assert m.calculate_admission_cost(list(range(8))).prefill_tokens == 1
    prefill(m, 2, list(range(8)))
    assert m.num_cached_tokens(2) == 8
    check_invariants(m)


def test_free_partial_page_is_attached_and_written_in_place():
    m = make()
    prefill(m, 1, list(range(10)))
    m.release(1)
    prompt = list(range(11))
    cost = m.calculate_admission_cost(prompt)
    assert (cost.blocks_needed, cost.prefill_tokens) == (3, 1)
    assert list(m.allocate(2, prompt)) == [0, 1, 2]
    assert m.num_cached_tokens(2) == 10 and not m.storage.copies


def test_shared_partial_page_is_copied_at_admission():
    m = make()
    prefill(m, 1, list(range(10)))
    m.release(1)
    prompt = list(range(11))
    m.allocate(2, prompt)
    cost = m.calculate_admission_cost(prompt)
    assert (cost.blocks_needed, cost.prefill_tokens) == (1, 1)
    table = list(m.allocate(3, prompt))
    assert table[:2] == [0, 1] and table[2] != 2
    assert m.storage.copies[-1] == (2, table[2], 2) and m.ref_counts[2] == 1


def test_partial_match_copies_only_what_matched():
    m = make()
    prefill(m, 1, list(range(10)))
    m.release(1)
    m.allocate(2, list(range(11)))
    prompt = list(range(8)) + [8, 99, 5]
    cost = m.calculate_admission_cost(prompt)
    assert (cost.blocks_needed, cost.prefill_tokens) == (1, 2)
    table = list(m.allocate(4, prompt))
    assert m.storage.copies[-1] == (2, table[2], 1) and m.num_cached_tokens(4) == 9


def test_free_copy_source_may_be_evicted_once_the_copy_is_made():
    m = make(2)
    prefill(m, 1, [1, 2, 3])
    m.release(1)
    prompt = [1, 2, 9, 9, 9, 9]
    cost = m.calculate_admission_cost(prompt)
    assert (cost.blocks_needed, cost.prefill_tokens) == (2, 4)
    assert list(m.allocate(2, prompt)) == [1, 0]
    assert m.storage.copies[-1] == (0, 1, 2) and 0 not in m.index


def test_copy_source_cannot_be_its_own_destination():
    m = make(2)
    prefill(m, 1, [1, 2, 3])
    m.release(1)
    m.allocate(2, [5, 5])
    assert m.calculate_admission_cost([1, 2, 9]).blocks_needed == 2 > m.num_available_blocks()
    assert m.allocate(3, [1, 2, 9]) is None


def test_refused_admission_changes_nothing():
    m = make(3)
    prefill(m, 1, list(range(10)))
    m.release(1)
    m.allocate(2, [50, 51, 52, 53, 54])
    sp = m.spaces[0]

    def snapshot():
        return (list(sp.holders), list(sp.idle), sp.kept, dict(sp.released_at), sorted(sp._queue), list(m.free_state_slots),
                {b: (m.index.tokens(b), m.index.parent(b)) for b in m.index}, set(m.seqs))

    before = snapshot()
    assert m.allocate(9, list(range(11))) is None
    assert snapshot() == before


def test_matched_pages_are_held_before_a_page_is_taken():
    m = make(3)
    prefill(m, 1, [1, 2, 3, 4, 5])
    m.release(1)
    prefill(m, 2, [7, 7])
    m.release(2)
    table = list(m.allocate(3, [1, 2, 3, 4, 6, 6, 6]))
    assert table[0] == 0 and 0 in m.index
    forward(m, 3)
    m.commit(3, 3)
    check_invariants(m)


def test_admitting_twice_is_refused():
    m = make()
    m.allocate(1, [1, 2])
    with pytest.raises(AssertionError):
        m.allocate(1, [3, 4])


def test_no_state_slot_no_admission():
    m = KVCacheManager(FakeStorage(12, (0,), state_slots=1))
    assert m.allocate(1, [1, 2]) is not None
    assert m.allocate(2, [3, 4]) is None and not m.can_fork()
    forward(m, 1)
    m.commit(1, 2)
    m.release(1)
    assert m.allocate(2, [3, 4]) is not None


# ---- free pool and eviction (tests/test_kvcache_manager.py:202-222) --------------------------------

def test_unpublished_pages_first_then_the_least_recently_freed_leaf():
    m = make(4)
    sp = m.spaces[0]
    b0, b1, b2, b3 = (sp.take() for _ in range(4))
    m.index.add(TOP, b0, [1, 2, 3, 4])
    m.index.add(b0, b1, [5, 6])
    m.index.add(TOP, b2, [9, 9, 9, 9])
    for b in (b3, b2, b0, b1):
        sp.drop(b)
    assert sp.idle == [3] and sp.kept == 3
    assert (sp.released_at[b2], sp.released_at[b0], sp.released_at[b1]) == (1, 2, 3)
    assert sp.take() == 3
    assert sp.take() == 2          # page 0 was released before page 1, but page 1 follows it
    assert 2 not in m.index and sp.kept == 2
    assert sp.take() == 1 and sp.take() == 0, "once nothing follows it, a page's turn comes by its own age"
    assert sp.available() == 0 and len(m.index) == 0


def test_free_pages_are_not_held_or_dropped_behind_the_pool():
    sp = make(2).spaces[0]
    b = sp.take()
    sp.drop(b)
    with pytest.raises(AssertionError):
        sp.hold(b)
    with pytest.raises(AssertionError):
        sp.drop(b)                 # freed twice


# ---- growing (tests/test_kvcache_manager.py:227-278) -----------------------------------------------

def test_append_fills_the_page_then_takes_one():
    m = make()
    prefill(m, 1, [1, 2, 3, 4, 5, 6])
    assert m.blocks_needed_for_append(1, 1) == 0
    step(m, 1, [7])
    step(m, 1, [8])
    assert m.seqs[1].block_table == [0, 1]
    assert m.blocks_needed_for_append(1, 1) == 1
    step(m, 1, [9])
    assert m.seqs[1].block_table == [0, 1, 2]
    check_invariants(m)


def test_append_needs_the_previous_step_committed_and_room():
    m = make()
    prefill(m, 1, [1, 2])
    m.append_slots(1, [3])
    with pytest.raises(AssertionError):
        m.append_slots(1, [4])
    m = make(1)
    prefill(m, 1, [1, 2, 3, 4])
    assert m.blocks_needed_for_append(1, 1) == 1 > m.num_available_blocks() and not m.can_append(1, 1)
    with pytest.raises(AssertionError):
        m.append_slots(1, [5])
    assert m.seqs[1].reserved == 4


def test_a_portion_takes_exactly_the_pages_it_predicts():
    m = make()
    prefill(m, 1, [1, 2, 3, 4, 5, 6])
    needed, before = m.blocks_needed_for_append(1, 7), m.num_available_blocks()
    m.append_slots(1, list(range(10, 17)))
    assert needed == 2 and before - m.num_available_blocks() == 2


def test_prompt_in_portions_equals_prompt_at_once():
    prompt = list(range(100, 123))
    whole, cut = make(), make()
    prefill(whole, 1, prompt)
    assert cut.calculate_admission_cost(prompt, feed=5).blocks_needed == 2
    prefill(cut, 1, prompt, feed=5)
    assert cut.seqs[1].committed == 5 and len(cut.seqs[1].block_table) == 2
    for a, b in ((5, 6), (6, 15), (15, 23)):
        step(cut, 1, prompt[a:b])
    assert cut.seqs[1].block_table == whole.seqs[1].block_table and cut.seqs[1].token_ids == prompt
    assert set(cut.index) == set(whole.index)
    check_invariants(cut)


def test_forks_copy_the_shared_tail_one_by_one():
    m = make()
    prefill(m, 1, [1, 2, 3, 4, 5])
    for c in (2, 3, 4):
        m.fork(1, c)
    needs = []
    for sid in (2, 3, 4, 1):
        needs.append(m.blocks_needed_for_append(sid, 1))
        step(m, sid, [10 * sid])
    assert needs == [1, 1, 1, 0]
    assert m.seqs[1].block_table == [0, 1] and m.ref_counts[:2] == [4, 1]
    assert m.stats().cow_copies == 3
    check_invariants(m)


def test_a_model_with_state_reuses_no_prefix():
    """A state slot starts empty at admission and is built only by the tokens that are fed: with
    prefix reuse the skipped tokens would be missing from it, so the manager turns reuse off by
    itself, also for a request that comes back after it gave up its pages."""
    m = make(keeps_state=True)
    assert not m.caching
    prefill(m, 1, list(range(10)))
    m.release(1)
    assert m.calculate_admission_cost(list(range(10))).prefill_tokens == 10
    prefill(m, 2, list(range(10)))
    assert m.num_cached_tokens(2) == 10 and m.storage.state[m.seqs[2].state_slot] == 45
    check_invariants(m)


def test_fork_copies_the_state_slot():
    m = make(keeps_state=True)
    prefill(m, 1, [1, 2, 3])
    m.fork(1, 2)
    assert m.seqs[2].state_slot != m.seqs[1].state_slot
    assert m.storage.state[m.seqs[2].state_slot] == 6
    step(m, 2, [10])
    step(m, 1, [20])
    check_invariants(m)
    m.release(1)
    m.release(2)
    assert len(m.free_state_slots) == m.storage.num_state_slots


# ---- commit, publish, dedupe (tests/test_kvcache_manager.py:283-360) -------------------------------

def test_commit_publishes_full_pages_only():
    m = make()
    prefill(m, 1, list(range(10)))
    assert set(m.index) == {0, 1}
    step(m, 1, [10])
    step(m, 1, [11])
    assert m.index.parent(2) == 1
    check_invariants(m)


def test_rejected_tokens_are_rolled_back():
    m = make()
    prefill(m, 1, list(range(10)))
    before = m.num_available_blocks()
    m.append_slots(1, list(range(10, 16)))
    forward(m, 1)
    m.storage.state[m.seqs[1].state_slot] -= sum(range(12, 16))
    m.commit(1, 2)
    s = m.seqs[1]
    assert s.committed == s.reserved == 12 and s.token_ids[-2:] == [10, 11]
    assert len(s.block_table) == 3 and m.num_available_blocks() == before
    check_invariants(m)
    step(m, 1, [99, 98])
    assert len(s.block_table) == 4 and s.token_ids[-2:] == [99, 98]
    check_invariants(m)


def test_over_accepting_is_refused_and_accepting_nothing_abandons_the_step():
    m = make()
    prefill(m, 1, [1, 2, 3])
    m.append_slots(1, [4, 5])
    with pytest.raises(AssertionError):
        m.commit(1, 3)
    m.commit(1, 0)
    assert m.seqs[1].committed == m.seqs[1].reserved == 3
    m.release(1)
    check_invariants(m)


def test_identical_prompts_run_together_are_deduplicated_at_commit():
    m = make()
    prompt = [1, 2, 3, 4, 5, 6, 7, 8, 9]
    m.allocate(1, prompt)
    m.allocate(2, prompt)
    for sid in (1, 2):
        forward(m, sid)
    m.commit(1, 9)
    m.commit(2, 9)
    assert m.seqs[2].block_table[:2] == m.seqs[1].block_table[:2]
    assert m.seqs[2].block_table[2] != m.seqs[1].block_table[2]
    assert m.stats().dedupes == 2
    check_invariants(m)


def test_release_stamps_deeper_pages_as_older():
    """tests/test_kvcache_manager.py:377-386: the tail is let go first, so it is evicted first."""
    m = make()
    prefill(m, 1, list(range(10)))
    m.release(1)
    stamps = [m.spaces[0].released_at[b] for b in (0, 1, 2)]
    assert stamps == sorted(stamps, reverse=True)
    check_invariants(m)


def test_caching_off_publishes_nothing_but_forks_still_share():
    m = make(caching=False)
    prefill(m, 1, list(range(10)))
    m.fork(1, 2)
    assert m.ref_counts[:3] == [2, 2, 2] and len(m.index) == 0
    m.release(1)
    m.release(2)
    assert m.num_available_blocks() == 12 and m.calculate_admission_cost(list(range(10))).prefill_tokens == 10
    check_invariants(m)


# ---- layers that read a window only --------------------------------------------------------------

def test_window_space_gives_pages_back_as_the_window_passes():
    m = make(pages=[12, 4], windows=(0, 6))
    assert not m.caching, "prefix reuse needs every layer's pages"
    prefill(m, 1, list(range(9)))
    s = m.seqs[1]
    # 9 committed, window 6: later tokens read positions >= 4, page 0 (0..3) is dead
    assert s.tables[1][0] == FREED and s.tables[1][1] != FREED and FREED not in s.tables[0]
    for t in range(9, 30):
        step(m, 1, [t])
        check_invariants(m)
        assert sum(p != FREED for p in s.tables[1]) <= 3
    assert m.stats().window_frees >= 5
    m.release(1)
    assert m.num_available_blocks(0) == 12 and m.num_available_blocks(1) == 4


def test_window_space_limits_admission():
    m = make(pages=[12, 2], windows=(0, 3))
    assert m.calculate_admission_cost(list(range(12))).per_space == (3, 3)
    assert m.allocate(1, list(range(12))) is None
    prefill(m, 1, list(range(12)), feed=8)
    step(m, 1, list(range(8, 12)))
    check_invariants(m)


# ---- random orders of requests -----------------------------------------------------------------------

@pytest.mark.parametrize("seed", range(12))
@pytest.mark.parametrize("setup", ["cached", "uncached", "windowed", "stateful"])
def test_random_workload_keeps_every_invariant(seed, setup):
    """Admissions in portions, decodes, multi-token appends with partial acceptance, forks,
    releases, in random order (after tests/test_kvcache_manager.py:577-618)."""
    rng = random.Random(seed)
    if setup == "windowed":
        m = make(pages=[16, 7], windows=(0, 5), keeps_state=True)
    else:
        # ("stateful" asks for prefix reuse as the engine does by default; the manager declines)
        m = make(pages=16, caching=setup != "uncached", keeps_state=setup != "cached")
    assert m.caching == (setup == "cached")
    families = [[rng.randrange(6) for _ in range(rng.randrange(2, 14))] for _ in range(4)]
    next_id, pending = 0, {}
    for _ in range(250):
        live = list(m.seqs)
        op = rng.random()
        if op < 0.3 or not live:
            prompt = rng.choice(families)[:rng.randrange(1, 14)] + [rng.randrange(6) for _ in range(rng.randrange(0, 5))]
            prompt = prompt or [1]
            feed = rng.choice([None, 1, 2, 5])
            if m.allocate(next_id, prompt, feed) is not None:
                s = m.seqs[next_id]
                forward(m, next_id)
                m.commit(next_id, s.reserved - s.committed)
                pending[next_id] = prompt[s.committed:]
                next_id += 1
        elif op < 0.7:
            sid = rng.choice(live)
            rest = pending.get(sid) or []
            n = rng.randrange(1, 4)
            tokens = rest[:n] if rest else [rng.randrange(6) for _ in range(n)]
            if m.can_append(sid, len(tokens)):
                accept = len(tokens) if rest else rng.randrange(0, len(tokens) + 1)
                m.append_slots(sid, tokens)
                forward(m, sid)
                if accept < len(tokens):
                    m.storage.state[m.seqs[sid].state_slot] -= sum(tokens[accept:])
                m.commit(sid, accept)
                pending[sid] = rest[len(tokens):]
        elif op < 0.8 and m.can_fork():
            sid = rng.choice(live)
            m.fork(sid, next_id)
            pending[next_id] = list(pending.get(sid) or [])
            next_id += 1
        else:
            sid = rng.choice(live)
            m.release(sid)
            pending.pop(sid, None)
        check_invariants(m)
    for sid in list(m.seqs):
        m.release(sid)
    check_invariants(m)
    for sp in m.spaces:
        assert sp.available() == sp.num_pages, "pages were lost"
    assert m.stats().blocks_in_use == 0

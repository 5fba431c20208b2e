"""The cache manager: which pages every live request holds, which pages are free, and which free
pages still hold reusable prefixes. Host-side bookkeeping only; the one device operation it
issues is a copy of a page's leading slots (tinyserve_llm/kvcache/manager.py:45-328).

What is kept from the reference: reference counts, block tables per request, token-granular
prefix reuse through the prefix index, copy-on-write of a shared tail page, publish/grow/dedupe at
commit, LRU eviction of free leaf pages, forks that share every page.

What is added:
  * page spaces. Layers whose mixers keep every key share space 0 (one page id addresses the
    pools of all of them); layers that only ever read a window of W positions get a space of
    their own, with their own page ids and block tables, and give a page back as soon as the
    window has passed it. Prefix reuse needs every layer's pages to be restorable, so it is only
    on when all layers are in space 0 and none keeps per-request state (a state slot is rebuilt only
    by feeding the tokens again).
  * portions. `allocate(..., feed=n)` reserves slots for the first n uncached tokens only; the
    rest of a prompt follows through `append_slots`, like decoded tokens.
  * a slot of fixed-size per-request state, taken at allocate, copied at fork, returned at
    release, for mixers that keep state instead of (or beside) keys.
"""

from __future__ import annotations

import heapq
from dataclasses import dataclass, field, replace
from typing import Protocol, Sequence

from tinyserve_llm_amd.cache.prefix_index import TOP, Hit, PrefixIndex

FREED = -1   # block-table entry of a page that a window has passed and that was given back


@dataclass(frozen=True)
class SpaceSpec:
    num_pages: int
    window: int = 0      # 0: every key stays; W: pages wholly older than the last W positions are freed


class Storage(Protocol):
    """What the manager needs of the memory it manages."""

    page_size: int
    spaces: Sequence[SpaceSpec]
    num_state_slots: int
    keeps_state: bool     # some layer folds every token it is fed into its request's state slot

    def copy_slots(self, space: int, src: int, dst: int, num_slots: int) -> None: ...
    def copy_state(self, src_slot: int, dst_slot: int) -> None: ...
    def reset_state(self, slot: int) -> None: ...


@dataclass
class SeqState:
    tables: list[list[int]]                  # per space: page ids in token order (FREED where given back)
    token_ids: list[int] = field(default_factory=list)   # one per reserved slot
    committed: int = 0                       # leading slots whose keys/values are written and accepted
    state_slot: int = -1

    @property
    def block_table(self) -> list[int]:
        return self.tables[0]

    @property
    def reserved(self) -> int:
        return len(self.token_ids)


@dataclass(frozen=True)
class AdmissionCost:
    blocks_needed: int                 # pages of space 0 the admission takes out of the free pool
    prefill_tokens: int                # prompt tokens that still have to go through the model
    per_space: tuple[int, ...] = ()    # the same count for every space


@dataclass
class CacheStats:
    """Running totals, plus two current values filled in by stats()."""
    evictions: int = 0
    cow_copies: int = 0
    partial_copies: int = 0
    publishes: int = 0
    dedupes: int = 0
    window_frees: int = 0
    blocks_in_use: int = 0
    cached_pages: int = 0


class PageSpace:
    """The page ids of one space and who has them. At any moment a page is in exactly one state:

      idle   nobody holds it and the prefix index does not know it: it lies on the `idle` stack
      kept   nobody holds it, but the index knows the tokens it holds: a later prompt may take it
             over, and once no indexed page follows it, it stands in the queue for eviction,
             oldest release first
      held   `holders[page]` requests have it in their tables (indexed or not)

    `take` hands out an idle page while there is one and evicts from the queue otherwise, so
    `available()` = idle + kept is what admission may count on. The queue is a heap of (moment of
    release, page) for kept pages that nothing follows; entries are not removed when a page is
    taken over or gets a follower, they are recognised as stale when they come up (the reference
    finds its victim by a scan over all cached pages, tinyserve_llm/kvcache/manager.py:85-100)."""

    def __init__(self, spec: SpaceSpec, page_size: int) -> None:
        self.num_pages = spec.num_pages
        self.window = spec.window
        self.holders = [0] * spec.num_pages
        self.idle = list(range(spec.num_pages - 1, -1, -1))    # pop() hands out page 0 first
        self.index = PrefixIndex(page_size)                    # stays empty unless pages are published
        self.kept = 0
        self.released_at: dict[int, int] = {}                  # kept page -> the moment its last holder let go
        self._queue: list[tuple[int, int]] = []
        self._moment = 0
        self.evictions = 0

    def available(self) -> int:
        return len(self.idle) + self.kept

    def take(self) -> int:
        """An unheld page for one holder; the caller has checked `available()`."""
        page = self.idle.pop() if self.idle else self._evict()
        assert self.holders[page] == 0
        self.holders[page] = 1
        return page

    def _evict(self) -> int:
        while self._queue:
            moment, page = heapq.heappop(self._queue)
            if self.released_at.get(page) == moment and self.index.is_leaf(page):     # else: stale
                before = self.index.parent(page)
                self.index.discard(page)
                del self.released_at[page]
                self.kept -= 1
                self.evictions += 1
                if before != TOP and before in self.released_at and self.index.is_leaf(before):
                    heapq.heappush(self._queue, (self.released_at[before], before))   # its turn comes by its own age
                return page
        raise AssertionError("no page to hand out: the caller must check available() first")

    def hold(self, page: int) -> None:
        """One more request has the page in its table (a kept page is taken over)."""
        if self.holders[page] == 0:
            assert page in self.released_at, "an idle page is handed out by take()"
            del self.released_at[page]
            self.kept -= 1
        self.holders[page] += 1

    def drop(self, page: int) -> None:
        """One request less has it; the last one's leaving makes it kept (if indexed) or idle."""
        assert self.holders[page] > 0, f"page {page} is freed twice"
        self.holders[page] -= 1
        if self.holders[page]:
            return
        if page not in self.index:
            self.idle.append(page)
            return
        self._moment += 1
        self.released_at[page] = self._moment
        self.kept += 1
        if self.index.is_leaf(page):
            heapq.heappush(self._queue, (self._moment, page))


class KVCacheManager:
    def __init__(self, storage: Storage, caching: bool = True) -> None:
        self.storage = storage
        self.block_size = storage.page_size
        self.spaces = [PageSpace(s, self.block_size) for s in storage.spaces]
        assert self.spaces, "a model without any cache still gets one (empty) space"
        # A reused prefix is never fed to the model again, so every layer must find what it keeps of
        # those tokens still in place: pages of a space without a window qualify; pages that a window
        # has given back do not, and neither does a state slot, which starts empty at admission and
        # is only ever built by feeding the tokens. A model with either runs every prompt in full.
        self.caching = (caching and len(self.spaces) == 1 and self.spaces[0].window == 0
                        and not storage.keeps_state)
        self.seqs: dict[int, SeqState] = {}
        self.free_state_slots = list(range(storage.num_state_slots - 1, -1, -1))
        self.counters = CacheStats()

    # ---- views ------------------------------------------------------------------------------
    @property
    def index(self) -> PrefixIndex:
        return self.spaces[0].index

    @property
    def num_blocks(self) -> int:
        return self.spaces[0].num_pages

    @property
    def ref_counts(self) -> list[int]:
        return self.spaces[0].holders

    def num_available_blocks(self, space: int = 0) -> int:
        return self.spaces[space].available()

    def fits(self, per_space: Sequence[int], reserve: int = 0) -> bool:
        """True if every space can give `per_space[i] + reserve` pages."""
        return all(need + reserve <= sp.available() for need, sp in zip(per_space, self.spaces))

    def num_cached_tokens(self, seq_id: int) -> int:
        return self.seqs[seq_id].committed

    def block_table(self, seq_id: int, space: int = 0) -> list[int]:
        return self.seqs[seq_id].tables[space]

    def state_slot(self, seq_id: int) -> int:
        return self.seqs[seq_id].state_slot

    # ---- admission --------------------------------------------------------------------------
    def _pages_for(self, tokens: int) -> int:
        return -(-tokens // self.block_size)

    def _lookup(self, token_ids: Sequence[int]) -> Hit:
        return self.index.lookup(token_ids) if self.caching else Hit()

    def _copy_source(self, hit: Hit) -> int | None:
        """The page whose leading slots a hit's tail is copied from: a held one if there is one
        (a kept one could be evicted to make room for the copy), the lowest id among equals."""
        if not hit.tail:
            return None
        holders = self.spaces[0].holders
        return min(hit.tail_holders, key=lambda page: (holders[page] == 0, page))

    def _cost(self, hit: Hit, source: int | None, num_tokens: int, feed: int | None) -> AdmissionCost:
        """Pages that leave `available()` of each space if the prompt is admitted on this hit."""
        main = self.spaces[0]
        uncached = num_tokens - hit.num_tokens
        fed = uncached if feed is None else min(feed, uncached)
        in_all = self._pages_for(hit.num_tokens + fed)
        fresh = in_all - len(hit.pages)                      # pages to take beyond the ones taken over
        last = hit.pages[-1] if hit.pages else None
        if last is not None and len(main.index.tokens(last)) < self.block_size and main.holders[last]:
            fresh += 1                                       # a shared page that is not full is copied before the first write
        if source is not None and not main.holders[source]:
            fresh = max(fresh, 2)                            # a kept source must survive until its copy exists
        kept_taken_over = sum(1 for page in hit.pages if not main.holders[page])
        first = fresh + kept_taken_over
        return AdmissionCost(first, uncached, (first, *(in_all for _ in self.spaces[1:])))

    def calculate_admission_cost(self, token_ids: Sequence[int], feed: int | None = None) -> AdmissionCost:
        """What admitting this prompt (its first `feed` uncached tokens) would take. Changes nothing."""
        hit = self._lookup(token_ids)
        return self._cost(hit, self._copy_source(hit), len(token_ids), feed)

    def allocate(self, seq_id: int, token_ids: Sequence[int], feed: int | None = None) -> list[int] | None:
        """Admits a request: attaches its cached prefix, copies a partial match, reserves slots
        for the first `feed` uncached tokens (all of them if None). Returns the block table of
        space 0, or None, with nothing changed, if pages or state slots do not suffice."""
        assert token_ids, "a prompt has at least one token"
        assert seq_id not in self.seqs, "request is already admitted"
        hit = self._lookup(token_ids)
        source = self._copy_source(hit)
        cost = self._cost(hit, source, len(token_ids), feed)
        if not self.fits(cost.per_space) or not self.free_state_slots:
            return None
        main = self.spaces[0]
        seq = SeqState(tables=[[] for _ in self.spaces])
        seq.state_slot = self.free_state_slots.pop()
        self.storage.reset_state(seq.state_slot)
        table = seq.tables[0]
        for page in hit.pages:            # taken over first: nothing taken below may evict them
            main.hold(page)
            table.append(page)
        if source is not None:
            main.hold(source)             # (held for the moment of the copy only)
            copy = main.take()
            self.storage.copy_slots(0, source, copy, hit.tail)
            self.counters.partial_copies += 1
            main.drop(source)
            table.append(copy)
        seq.committed = hit.num_tokens
        seq.token_ids = list(token_ids[:seq.committed])
        uncached = token_ids[seq.committed:]
        self._reserve(seq, uncached if feed is None else uncached[:feed])
        self.seqs[seq_id] = seq
        return table

    # ---- growing ----------------------------------------------------------------------------
    def _reserve(self, seq: SeqState, token_ids: Sequence[int]) -> None:
        used_in_last = seq.reserved % self.block_size
        want_pages = self._pages_for(seq.reserved + len(token_ids))
        for index, (space, table) in enumerate(zip(self.spaces, seq.tables)):
            if used_in_last and token_ids:
                last = table[-1]
                if space.holders[last] > 1:    # shared tail: copy before the first write
                    fresh = space.take()
                    self.storage.copy_slots(index, last, fresh, used_in_last)
                    self.counters.cow_copies += 1
                    space.drop(last)
                    table[-1] = fresh
                else:
                    assert last not in space.index or used_in_last >= len(space.index.tokens(last)), \
                        "a published slot would be overwritten"
            while len(table) < want_pages:
                table.append(space.take())
        seq.token_ids.extend(token_ids)

    def blocks_needed_for_append(self, seq_id: int, num_tokens: int, space: int = 0) -> int:
        seq = self.seqs[seq_id]
        table = seq.tables[space]
        need = self._pages_for(seq.reserved + num_tokens) - len(table)
        if num_tokens and seq.reserved % self.block_size and self.spaces[space].holders[table[-1]] > 1:
            need += 1      # the shared tail page is copied first
        return need

    def can_append(self, seq_id: int, num_tokens: int) -> bool:
        seq = self.seqs[seq_id]
        if num_tokens and (seq.reserved % self.block_size) + num_tokens <= self.block_size and seq.reserved % self.block_size:
            # the tokens stay inside the last page: pages are needed only to copy a shared tail
            return all(sp.holders[t[-1]] <= 1 or sp.available() >= 1 for sp, t in zip(self.spaces, seq.tables))
        return all(self.blocks_needed_for_append(seq_id, num_tokens, i) <= sp.available()
                   for i, sp in enumerate(self.spaces))

    def append_slots(self, seq_id: int, token_ids: Sequence[int], checked: bool = False) -> None:
        """Reserves slots for the tokens a step feeds to an admitted request: a decoded token or the
        next portion of its prompt. Closed by commit(). `checked`: the caller has just asked
        can_append for this very request and count."""
        assert token_ids, "a step feeds at least one token"
        seq = self.seqs[seq_id]
        assert seq.reserved == seq.committed, "the previous step was not committed"
        assert checked or self.can_append(seq_id, len(token_ids)), "not enough free pages; preempt first"
        self._reserve(seq, token_ids)

    def try_append_one(self, seq_id: int, token: int) -> bool:
        """`can_append` and `append_slots` for the one token of a decoding request, in one pass
        (a step of hundreds of requests asks this for every one of them): reserves the slot and
        returns True, or changes nothing and returns False where pages are missing."""
        seq = self.seqs[seq_id]
        reserved = len(seq.token_ids)
        assert reserved == seq.committed, "the previous step was not committed"
        used_in_last = reserved % self.block_size
        for space, table in zip(self.spaces, seq.tables):       # first pass: is there room everywhere
            if used_in_last:
                if space.holders[table[-1]] > 1 and space.available() < 1:
                    return False
            elif self._pages_for(reserved + 1) > len(table) and space.available() < 1:
                return False
        self._reserve(seq, (token,))
        return True

    def set_token(self, seq_id: int, position: int, token: int) -> None:
        """Names the token of a reserved, not yet committed slot whose token was not known when the
        slot was reserved (pages are published by their tokens, at commit)."""
        seq = self.seqs[seq_id]
        assert seq.committed <= position < seq.reserved, "only a reserved slot can still be named"
        seq.token_ids[position] = token

    def commit(self, seq_id: int, num_accepted: int) -> None:
        """Closes a step: keeps the first `num_accepted` slots reserved since the last commit,
        drops the rest, publishes pages that became full, frees pages a window has passed."""
        seq = self.seqs[seq_id]
        assert 0 <= num_accepted <= seq.reserved - seq.committed, "more slots accepted than reserved"
        before = seq.committed
        seq.committed += num_accepted
        del seq.token_ids[seq.committed:]
        keep = self._pages_for(seq.committed)
        for space, table in zip(self.spaces, seq.tables):
            while len(table) > keep:
                page = table.pop()
                if page != FREED:
                    space.drop(page)
        if self.caching:
            for i in range(before // self.block_size, seq.committed // self.block_size):
                self._publish(seq, i)
        for space, table in zip(self.spaces, seq.tables):
            if space.window:
                self._free_passed(space, table, seq.committed)

    def _free_passed(self, space: PageSpace, table: list[int], committed: int) -> None:
        """A later token sits at position >= committed and reads keys > position - window: page j
        (positions j*bs .. (j+1)*bs - 1) is dead once (j+1)*bs <= committed - window + 1."""
        dead = max(0, min(len(table), (committed - space.window + 1) // self.block_size))
        for j in range(dead - 1, -1, -1):
            if table[j] == FREED:
                break
            space.drop(table[j])
            table[j] = FREED
            self.counters.window_frees += 1

    def _publish(self, seq: SeqState, i: int) -> None:
        """Makes page i of the request findable by the tokens committed into it. If the index has
        a page with these very tokens after the same page already, the request moves over to that
        one and lets its own go."""
        main, table = self.spaces[0], seq.tables[0]
        page, index = table[i], main.index
        tokens = seq.token_ids[i * self.block_size:min((i + 1) * self.block_size, seq.committed)]
        if page not in index:
            stands = index.add(table[i - 1] if i else TOP, page, tokens)
            self.counters.publishes += stands == page
        elif len(index.tokens(page)) < len(tokens):
            stands = index.extend(page, tokens)       # a page taken over while it was not full, written further into
        else:
            return
        if stands != page:
            self.counters.dedupes += 1
            main.hold(stands)
            table[i] = stands
            main.drop(page)

    # ---- leaving, forking -------------------------------------------------------------------
    def release(self, seq_id: int) -> None:
        """Drops a finished or preempted request. Its pages stay in the tree for later prompts;
        they are let go tail first, so that deeper pages look older and are evicted first."""
        seq = self.seqs[seq_id]
        assert seq.reserved == seq.committed, "commit before release"
        if self.caching and seq.committed % self.block_size:
            self._publish(seq, seq.committed // self.block_size)
        del self.seqs[seq_id]
        for space, table in zip(self.spaces, seq.tables):
            for page in reversed(table):
                if page != FREED:
                    space.drop(page)
        self.free_state_slots.append(seq.state_slot)

    def can_fork(self) -> bool:
        return bool(self.free_state_slots)

    def fork(self, src_id: int, new_id: int) -> None:
        """Starts `new_id` as a copy of `src_id` that shares all its pages (the tail too: whoever
        writes first copies it) and has a copy of its state."""
        assert new_id not in self.seqs, "request is already admitted"
        src = self.seqs[src_id]
        assert src.reserved == src.committed, "commit before fork"
        assert self.free_state_slots, "no state slot left for the fork"
        for space, table in zip(self.spaces, src.tables):
            for page in table:
                if page != FREED:
                    space.hold(page)
        slot = self.free_state_slots.pop()
        self.storage.copy_state(src.state_slot, slot)
        self.seqs[new_id] = SeqState(tables=[list(t) for t in src.tables], token_ids=list(src.token_ids),
                                     committed=src.committed, state_slot=slot)

    def stats(self) -> CacheStats:
        main = self.spaces[0]
        return replace(self.counters, evictions=sum(s.evictions for s in self.spaces),
                       blocks_in_use=main.num_pages - main.available(), cached_pages=len(main.index))

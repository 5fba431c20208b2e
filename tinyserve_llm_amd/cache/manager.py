"""The cache manager: which pages every live request holds, which pages are free, and which free
pages still hold reusable prefixes. Host-side bookkeeping only; the one device operation it
issues is a copy of a page's leading slots (tinyserve_llm/kvcache/manager.py:45-328).

What is kept from the reference: reference counts, block tables per request, token-granular
prefix reuse through the page tree, copy-on-write of a shared tail page, publish/grow/dedupe at
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

from dataclasses import dataclass, field, replace
from typing import Protocol, Sequence

from tinyserve_llm_amd.cache.page_tree import Match, PageNode, PageTree

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
    """Reference counts, the free list and (for space 0) the prefix tree of one set of page ids."""

    def __init__(self, spec: SpaceSpec, page_size: int) -> None:
        self.num_pages = spec.num_pages
        self.window = spec.window
        self.refs = [0] * spec.num_pages
        self.free = list(range(spec.num_pages - 1, -1, -1))   # pop() hands out page 0 first
        self.tree = PageTree(page_size)                        # stays empty unless pages are published
        self.free_cached = 0                                   # published pages nobody holds
        self.clock = 0
        self.evictions = 0

    def available(self) -> int:
        return len(self.free) + self.free_cached

    def take(self) -> int:
        """A page with one holder: a never-published free one if there is one, else the least
        recently released free leaf of the tree."""
        page = self.free.pop() if self.free else self._evict()
        assert self.refs[page] == 0
        self.refs[page] = 1
        return page

    def _evict(self) -> int:
        victim = min((n for n in self.tree.nodes.values() if self.refs[n.block_id] == 0 and not n.children),
                     key=lambda n: n.last_used, default=None)
        assert victim is not None, "no free page: the caller must check available() first"
        self.free_cached -= 1
        self.evictions += 1
        return self.tree.evict(victim)

    def hold(self, page: int) -> None:
        if self.refs[page] == 0:
            assert page in self.tree.nodes, "a free unpublished page is handed out by take()"
            self.free_cached -= 1
        self.refs[page] += 1

    def drop(self, page: int) -> None:
        assert self.refs[page] > 0, f"page {page} is freed twice"
        self.refs[page] -= 1
        if self.refs[page]:
            return
        node = self.tree.nodes.get(page)
        if node is None:
            self.free.append(page)
        else:
            self.clock += 1
            node.last_used = self.clock
            self.free_cached += 1


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
    def tree(self) -> PageTree:
        return self.spaces[0].tree

    @property
    def num_blocks(self) -> int:
        return self.spaces[0].num_pages

    @property
    def ref_counts(self) -> list[int]:
        return self.spaces[0].refs

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

    def _match(self, token_ids: Sequence[int]) -> Match:
        return self.tree.match(token_ids) if self.caching else Match([])

    def _partial_source(self, match: Match) -> PageNode | None:
        """The page to copy a partial match from; one that is in use is preferred, because it
        cannot be evicted while the destination is taken."""
        if not match.partial_len:
            return None
        refs = self.spaces[0].refs
        return min(match.partial_candidates, key=lambda p: refs[p.block_id] == 0)

    def _cost(self, match: Match, source: PageNode | None, num_tokens: int, feed: int | None) -> AdmissionCost:
        uncached = num_tokens - match.num_tokens
        now = uncached if feed is None else min(feed, uncached)
        cover = match.num_tokens + now
        refs, pages = self.spaces[0].refs, match.pages
        take = self._pages_for(cover) - len(pages)
        # the last attached page is partial and somebody holds it: writing past it copies it first
        if pages and len(pages[-1].tokens) < self.block_size and refs[pages[-1].block_id] > 0:
            take += 1
        # copying out of a free page: source and destination must exist side by side
        if source is not None and refs[source.block_id] == 0:
            take = max(take, 2)
        # attached pages that were free leave the free pool too
        take += sum(1 for p in pages if refs[p.block_id] == 0)
        rest = tuple(self._pages_for(cover) for _ in self.spaces[1:])
        return AdmissionCost(take, uncached, (take, *rest))

    def calculate_admission_cost(self, token_ids: Sequence[int], feed: int | None = None) -> AdmissionCost:
        """What admitting this prompt (its first `feed` uncached tokens) would take. Changes nothing."""
        match = self._match(token_ids)
        return self._cost(match, self._partial_source(match), len(token_ids), feed)

    def allocate(self, seq_id: int, token_ids: Sequence[int], feed: int | None = None) -> list[int] | None:
        """Admits a request: attaches its cached prefix, copies a partial match, reserves slots
        for the first `feed` uncached tokens (all of them if None). Returns the block table of
        space 0, or None, with nothing changed, if pages or state slots do not suffice."""
        assert token_ids, "a prompt has at least one token"
        assert seq_id not in self.seqs, "request is already admitted"
        match = self._match(token_ids)
        source = self._partial_source(match)
        cost = self._cost(match, source, len(token_ids), feed)
        if not self.fits(cost.per_space) or not self.free_state_slots:
            return None
        main = self.spaces[0]
        seq = SeqState(tables=[[] for _ in self.spaces])
        seq.state_slot = self.free_state_slots.pop()
        self.storage.reset_state(seq.state_slot)
        table = seq.tables[0]
        for page in match.pages:          # hold what matched before anything is taken or evicted
            main.hold(page.block_id)
            table.append(page.block_id)
        if source is not None:
            main.hold(source.block_id)
            dest = main.take()
            self.storage.copy_slots(0, source.block_id, dest, match.partial_len)
            self.counters.partial_copies += 1
            main.drop(source.block_id)
            table.append(dest)
        seq.committed = match.num_tokens
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
                if space.refs[last] > 1:       # shared tail: copy before the first write
                    fresh = space.take()
                    self.storage.copy_slots(index, last, fresh, used_in_last)
                    self.counters.cow_copies += 1
                    space.drop(last)
                    table[-1] = fresh
                else:
                    node = space.tree.nodes.get(last)
                    assert node is None or used_in_last >= len(node.tokens), "a published slot would be overwritten"
            while len(table) < want_pages:
                table.append(space.take())
        seq.token_ids.extend(token_ids)

    def blocks_needed_for_append(self, seq_id: int, num_tokens: int, space: int = 0) -> int:
        seq = self.seqs[seq_id]
        table = seq.tables[space]
        need = self._pages_for(seq.reserved + num_tokens) - len(table)
        if num_tokens and seq.reserved % self.block_size and self.spaces[space].refs[table[-1]] > 1:
            need += 1      # the shared tail page is copied first
        return need

    def can_append(self, seq_id: int, num_tokens: int) -> bool:
        seq = self.seqs[seq_id]
        if num_tokens and (seq.reserved % self.block_size) + num_tokens <= self.block_size and seq.reserved % self.block_size:
            # the tokens stay inside the last page: pages are needed only to copy a shared tail
            return all(sp.refs[t[-1]] <= 1 or sp.available() >= 1 for sp, t in zip(self.spaces, seq.tables))
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
                if space.refs[table[-1]] > 1 and space.available() < 1:
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
        """Records page i of the request in the tree under the page before it; swaps to an
        identical page if the tree already has one."""
        main, table = self.spaces[0], seq.tables[0]
        page = table[i]
        parent = main.tree.nodes[table[i - 1]] if i else main.tree.root
        tokens = seq.token_ids[i * self.block_size:min((i + 1) * self.block_size, seq.committed)]
        node = main.tree.nodes.get(page)
        if node is None:
            kept = main.tree.publish(parent, page, tokens)
            if kept.block_id == page:
                self.counters.publishes += 1
        elif len(node.tokens) < len(tokens):
            assert node.parent is parent
            kept = main.tree.grow(node, tokens)      # an attached partial page we wrote further into
        else:
            return
        if kept.block_id != page:
            self.counters.dedupes += 1
            main.hold(kept.block_id)
            table[i] = kept.block_id
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
                       blocks_in_use=main.num_pages - main.available(), cached_pages=len(main.tree.nodes))

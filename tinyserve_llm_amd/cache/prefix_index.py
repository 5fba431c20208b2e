"""The prefix index: which pages of the cache hold which runs of tokens, so that a new prompt can
take over the pages of its longest cached prefix, down to a single token inside a page. It plays
the part of the reference's page tree (tinyserve_llm/kvcache/page_tree.py:8-127: publish, grow,
match, evict, with a token trie under every page); the structure here is one table and one kind of
index:

  * a table from page id to what the page holds: its tokens, the page before it, how many pages
    follow it;
  * under every page (and under the start of all prompts, page id TOP) a token trie over the runs
    of the pages that follow it. The trie answers both questions a lookup has: which page holds
    exactly this run (the trie marks where a run ends), and which pages share the longest
    beginning of it. There is no second table of children by their tokens.

Pages are named by their ids throughout; the index keeps no reference counts and no ages (the
page space that owns the ids does).
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Iterator, Sequence

from tinyserve_llm_amd.cache.trie import TokenTrie

TOP = -1     # stands for "before the first page": the parent of every prompt's first page


@dataclass
class Hit:
    """What a lookup found. `pages` are taken over as they are (every token they hold matches);
    after them, `tail` more tokens match the beginning of each page in `tail_holders`, which a
    caller may copy from."""

    pages: list[int] = field(default_factory=list)
    covered: int = 0                              # tokens held by `pages`
    tail: int = 0
    tail_holders: frozenset[int] = frozenset()

    @property
    def num_tokens(self) -> int:
        return self.covered + self.tail


class _Entry:
    __slots__ = ("tokens", "parent", "followers", "below")

    def __init__(self, tokens: tuple[int, ...], parent: int) -> None:
        self.tokens = tokens                      # what the page holds; only ever gets longer
        self.parent = parent
        self.followers = 0                        # pages indexed under this one
        self.below: TokenTrie | None = None       # their runs; made when the first one arrives


class PrefixIndex:
    def __init__(self, page_size: int) -> None:
        self.page_size = page_size
        self._entries: dict[int, _Entry] = {}
        self._top = TokenTrie()

    # ---- reading ----------------------------------------------------------------------------------
    def __contains__(self, page: int) -> bool:
        return page in self._entries

    def __len__(self) -> int:
        return len(self._entries)

    def __iter__(self) -> Iterator[int]:
        return iter(self._entries)

    def tokens(self, page: int) -> tuple[int, ...]:
        return self._entries[page].tokens

    def parent(self, page: int) -> int:
        return self._entries[page].parent

    def is_leaf(self, page: int) -> bool:
        return self._entries[page].followers == 0

    def _under(self, page: int) -> TokenTrie | None:
        return self._top if page == TOP else self._entries[page].below

    def lookup(self, token_ids: Sequence[int]) -> Hit:
        """The longest cached prefix of `token_ids` short of its last token, which has to go through
        the model to give the first logits (the reference stops there too, page_tree.py:47)."""
        stop = len(token_ids) - 1
        hit = Hit()
        at = TOP
        while hit.covered < stop:
            trie = self._under(at)
            if trie is None:
                break
            run = tuple(token_ids[hit.covered:min(hit.covered + self.page_size, stop)])
            depth, holders, exact = trie.find(run)
            if depth == 0:
                break
            if exact is None:
                # no page holds just these `depth` tokens; those that begin with them can be copied from
                hit.tail, hit.tail_holders = depth, frozenset(holders)
                break
            hit.pages.append(exact)
            hit.covered += depth
            if depth < len(run):
                break                             # a page that is not full has nothing after it
            at = exact
        return hit

    # ---- writing ----------------------------------------------------------------------------------
    def add(self, parent: int, page: int, tokens: Sequence[int]) -> int:
        """Enters `page`, holding `tokens`, after `parent` (TOP for a prompt's first page). Returns
        the page that stands for this run from now on: `page`, or the one that was there already."""
        run = tuple(tokens)
        if not 0 < len(run) <= self.page_size:
            raise AssertionError(f"a page holds 1 to {self.page_size} tokens, not {len(run)}")
        if page in self._entries:
            raise AssertionError(f"page {page} is indexed already; extend it")
        if parent != TOP and len(self._entries[parent].tokens) != self.page_size:
            raise AssertionError("only a full page is followed by another")
        trie = self._under(parent)
        if trie is None:
            trie = self._entries[parent].below = TokenTrie()
        there = trie.exact(run)
        if there is not None:
            return there
        trie.insert(page, run)
        self._entries[page] = _Entry(run, parent)
        if parent != TOP:
            self._entries[parent].followers += 1
        return page

    def extend(self, page: int, tokens: Sequence[int]) -> int:
        """`page` now holds `tokens`, which begin with what it held. Returns the page that stands
        for the longer run: `page`, or a neighbour that held it already (then `page` stays as it was)."""
        run, entry = tuple(tokens), self._entries[page]
        if not len(entry.tokens) < len(run) <= self.page_size or run[:len(entry.tokens)] != entry.tokens:
            raise AssertionError("a page is extended by tokens after its own")
        trie = self._under(entry.parent)
        there = trie.exact(run)
        if there is not None:
            return there
        trie.insert(page, run)                    # walks the old path again and goes on from its end
        entry.tokens = run
        return page

    def discard(self, page: int) -> None:
        """Takes a page that nothing follows out of the index."""
        entry = self._entries[page]
        if entry.followers:
            raise AssertionError("a page that others follow stays")
        self._under(entry.parent).remove(page, entry.tokens)
        del self._entries[page]
        if entry.parent != TOP:
            self._entries[entry.parent].followers -= 1

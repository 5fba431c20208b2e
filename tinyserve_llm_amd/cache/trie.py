"""A trie over the token runs of one page's child pages, for token-granular prefix lookup
(tinyserve_llm/kvcache/trie.py:9-68). A trie node remembers every child page whose tokens pass
through it, so the deepest node reached names all pages that share the matched run."""

from __future__ import annotations

from typing import Hashable, Iterable, Sequence


class _Node:
    __slots__ = ("next", "pages")

    def __init__(self) -> None:
        self.next: dict[int, _Node] = {}
        self.pages: set = set()


class TokenTrie:
    __slots__ = ("root",)

    def __init__(self) -> None:
        self.root = _Node()

    def insert(self, page: Hashable, tokens: Sequence[int]) -> None:
        """Records `page` along the path of `tokens`. Inserting a longer run of a page already
        present walks its old path again (adding nothing there) and extends it."""
        if not tokens:
            raise AssertionError("a page in the trie holds at least one token")
        at = self.root
        for tok in tokens:
            nxt = at.next.get(tok)
            if nxt is None:
                nxt = at.next[tok] = _Node()
            nxt.pages.add(page)
            at = nxt

    def remove(self, page: Hashable, tokens: Sequence[int]) -> None:
        """Takes `page` off its path and prunes the part of the path nobody else uses."""
        at = self.root
        for tok in tokens:
            nxt = at.next[tok]
            nxt.pages.remove(page)
            if not nxt.pages:
                del at.next[tok]   # everything below belonged to this page alone
                return
            at = nxt

    def longest_match(self, tokens: Iterable[int]) -> tuple[int, set]:
        """(number of leading tokens found, the pages at the deepest node). The set is the trie's
        own: read it, do not change it."""
        at, depth = self.root, 0
        for tok in tokens:
            nxt = at.next.get(tok)
            if nxt is None:
                break
            at, depth = nxt, depth + 1
        return depth, at.pages

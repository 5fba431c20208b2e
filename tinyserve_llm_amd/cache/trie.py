"""A trie over the token runs of one page's child pages, for token-granular prefix lookup
(tinyserve_llm/kvcache/trie.py:9-68). A position in the trie remembers every child page whose
tokens pass through it, so the deepest position reached names all pages that share the matched run.

Runs of tokens that no other page leaves are kept as one edge (a page of 256 tokens that shares
nothing with its siblings is one node, not 256): an edge carries its tokens as a tuple and the set
of pages that pass through it, and every page that enters an edge reaches its end, because a run
that ends inside an edge splits the edge there. All positions inside an edge therefore see the same
pages, the set of the node at the edge's end. The node where a page's run ends is marked with that
page, so the page that holds exactly a given run is found by the same walk (two pages never hold
the same run: the index above swaps to the first)."""

from __future__ import annotations

from typing import Hashable, Iterable, Sequence


class _Node:
    __slots__ = ("label", "next", "pages", "ends")

    def __init__(self, label: tuple[int, ...] = (), pages: set | None = None) -> None:
        self.label = label                       # the tokens from the parent to here; empty for the root only
        self.next: dict[int, _Node] = {}         # first token of an edge -> the node at its end
        self.pages: set = set() if pages is None else pages
        self.ends: Hashable | None = None        # the page whose run ends exactly here


def _shared(label: tuple[int, ...], tokens: tuple[int, ...], at: int) -> int:
    """How many leading tokens of `label` equal tokens[at:]."""
    n = min(len(label), len(tokens) - at)
    if tokens[at:at + n] == label[:n]:
        return n
    m = 0
    while label[m] == tokens[at + m]:
        m += 1
    return m


class TokenTrie:
    __slots__ = ("root",)

    def __init__(self) -> None:
        self.root = _Node()

    @staticmethod
    def _split(parent: _Node, node: _Node, m: int) -> _Node:
        """Cuts the edge into `node` after m of its tokens; returns the new node at the cut."""
        upper = _Node(node.label[:m], set(node.pages))
        node.label = node.label[m:]
        upper.next[node.label[0]] = node
        parent.next[upper.label[0]] = upper
        return upper

    def insert(self, page: Hashable, tokens: Sequence[int]) -> None:
        """Records `page` along the path of `tokens`. Inserting a longer run of a page already
        present walks its old path again (adding nothing there) and extends it."""
        if not tokens:
            raise AssertionError("a page in the trie holds at least one token")
        run = tuple(tokens)
        at, i = self.root, 0
        while i < len(run):
            nxt = at.next.get(run[i])
            if nxt is None:
                nxt = at.next[run[i]] = _Node(run[i:], {page})
                nxt.ends = page
                return
            m = _shared(nxt.label, run, i)
            if m < len(nxt.label):           # the run leaves the edge, or ends inside it
                nxt = self._split(at, nxt, m)
            nxt.pages.add(page)
            if nxt.ends == page:
                nxt.ends = None              # its shorter run ended here; the longer one goes on
            at, i = nxt, i + m
        at.ends = page

    def remove(self, page: Hashable, tokens: Sequence[int]) -> None:
        """Takes `page` off its path (`tokens` is the run it was last inserted with) and prunes
        the part of the path nobody else uses."""
        at, i = self.root, 0
        while i < len(tokens):
            nxt = at.next[tokens[i]]
            nxt.pages.remove(page)
            if nxt.ends == page:
                nxt.ends = None
            if not nxt.pages:
                del at.next[tokens[i]]   # everything below belonged to this page alone
                return
            at, i = nxt, i + len(nxt.label)

    def find(self, tokens: Iterable[int]) -> tuple[int, set, Hashable | None]:
        """(number of leading tokens found, the pages at the deepest position, the page whose run is
        exactly those tokens or None). The set is the trie's own: read it, do not change it."""
        run = tokens if isinstance(tokens, tuple) else tuple(tokens)
        at, depth = self.root, 0
        while depth < len(run):
            nxt = at.next.get(run[depth])
            if nxt is None:
                break
            m = _shared(nxt.label, run, depth)
            if m < len(nxt.label):
                return depth + m, nxt.pages, None          # inside an edge no run ends
            at, depth = nxt, depth + m
        return depth, at.pages, at.ends

    def longest_match(self, tokens: Iterable[int]) -> tuple[int, set]:
        """(number of leading tokens found, the pages at the deepest position)."""
        return self.find(tokens)[:2]

    def exact(self, tokens: Iterable[int]) -> Hashable | None:
        """The page whose run is exactly `tokens`, or None."""
        run = tokens if isinstance(tokens, tuple) else tuple(tokens)
        depth, _, page = self.find(run)
        return page if depth == len(run) else None

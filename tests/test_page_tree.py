"""Token trie and page tree on their own, with the cases the reference's tests pin
(tests/test_page_tree.py:12-120, page size 8)."""

import pytest

from tinyserve_llm_amd.cache.page_tree import PageTree
from tinyserve_llm_amd.cache.trie import TokenTrie

B = 8
FULL = list(range(100, 108))


def test_trie_returns_every_page_at_the_deepest_node():
    trie, p, q = TokenTrie(), object(), object()
    trie.insert(p, [1, 2, 3])
    trie.insert(q, [1, 2, 9])
    assert trie.longest_match([1, 2, 3, 4]) == (3, {p})
    assert trie.longest_match([1, 2, 7]) == (2, {p, q})
    assert trie.longest_match([5]) == (0, trie.root.pages)


def test_trie_remove_keeps_shared_paths_and_prunes_the_rest():
    trie, p, q = TokenTrie(), object(), object()
    trie.insert(p, [1, 2, 3])
    trie.insert(q, [1, 2, 9])
    trie.remove(p, [1, 2, 3])
    assert trie.longest_match([1, 2, 3]) == (2, {q})
    trie.remove(q, [1, 2, 9])
    assert not trie.root.next


def test_trie_insert_of_a_longer_run_extends_the_old_path():
    trie, p = TokenTrie(), object()
    trie.insert(p, [1, 2])
    trie.insert(p, [1, 2, 3, 4])
    assert trie.longest_match([1, 2, 3, 4, 5]) == (4, {p})
    trie.remove(p, [1, 2, 3, 4])
    assert not trie.root.next


class PerTokenTrie:
    """One node per token, as the reference keeps it (tinyserve_llm/kvcache/trie.py:9-68): the
    meaning that the trie's edges of several tokens must keep."""

    def __init__(self):
        self.root = ({}, set())

    def insert(self, page, tokens):
        at = self.root
        for tok in tokens:
            at = at[0].setdefault(tok, ({}, set()))
            at[1].add(page)

    def remove(self, page, tokens):
        at = self.root
        for tok in tokens:
            nxt = at[0][tok]
            nxt[1].remove(page)
            if not nxt[1]:
                del at[0][tok]
                return
            at = nxt

    def longest_match(self, tokens):
        at, depth = self.root, 0
        for tok in tokens:
            if tok not in at[0]:
                break
            at, depth = at[0][tok], depth + 1
        return depth, at[1]


@pytest.mark.parametrize("seed", range(6))
def test_trie_with_edges_of_several_tokens_answers_as_one_node_per_token_does(seed):
    """Random inserts, extensions, removals and lookups over a small alphabet, so that runs share
    prefixes, end inside each other and split each other's edges."""
    import random
    rng = random.Random(seed)
    trie, plain, runs = TokenTrie(), PerTokenTrie(), {}
    for step in range(600):
        what = rng.random()
        if what < 0.4 or not runs:
            page, run = object(), [rng.randrange(3) for _ in range(rng.randint(1, 9))]
            runs[page] = run
            trie.insert(page, run), plain.insert(page, run)
        elif what < 0.55:
            page = rng.choice(list(runs))
            runs[page] = runs[page] + [rng.randrange(3) for _ in range(rng.randint(1, 4))]
            trie.insert(page, runs[page]), plain.insert(page, runs[page])
        elif what < 0.8:
            page = rng.choice(list(runs))
            run = runs.pop(page)
            trie.remove(page, run), plain.remove(page, run)
        probe = tuple(rng.randrange(3) for _ in range(rng.randint(0, 12)))
        assert trie.longest_match(probe) == plain.longest_match(probe), f"step {step}: {probe}"
        for page, run in runs.items():
            depth, pages = trie.longest_match(run)
            assert depth == len(run) and page in pages
    for page, run in list(runs.items()):
        trie.remove(page, run)
    assert not trie.root.next and not trie.root.pages


def test_a_page_that_shares_nothing_is_one_edge():
    trie, p, q = TokenTrie(), object(), object()
    trie.insert(p, list(range(256)))
    assert len(trie.root.next) == 1 and not trie.root.next[0].next
    trie.insert(q, list(range(100)) + [7])
    upper = trie.root.next[0]
    assert len(upper.label) == 100 and upper.pages == {p, q} and set(upper.next) == {100, 7}


def test_publish_returns_the_twin_on_a_duplicate():
    t = PageTree(B)
    a = t.publish(t.root, 1, FULL)
    assert a.block_id == 1 and t.nodes == {1: a}
    assert t.publish(t.root, 2, FULL) is a and 2 not in t.nodes


def test_publish_needs_a_full_parent_and_a_new_page():
    t = PageTree(B)
    partial = t.publish(t.root, 1, [7, 7])
    with pytest.raises(AssertionError):
        t.publish(partial, 2, [1])
    a = t.publish(t.root, 3, FULL)
    with pytest.raises(AssertionError):
        t.publish(a, 3, [1])


def test_match_walks_full_pages_and_attaches_an_exact_partial_page():
    t = PageTree(B)
    a = t.publish(t.root, 1, FULL)
    c = t.publish(a, 2, [1, 2, 3])
    m = t.match(FULL + [1, 2, 3, 99])
    assert m.pages == [a, c] and m.partial_len == 0 and m.num_tokens == 11


def test_match_reports_a_partial_run_with_its_holders():
    t = PageTree(B)
    a = t.publish(t.root, 1, FULL)
    c = t.publish(a, 2, [1, 2, 3])
    m = t.match(FULL + [1, 2, 9, 9])
    assert m.pages == [a] and m.partial_len == 2 and m.partial_candidates == {c} and m.num_tokens == 10


def test_match_never_covers_the_last_token():
    t = PageTree(B)
    a = t.publish(t.root, 1, FULL)
    m = t.match(FULL)
    assert m.pages == [] and m.partial_len == B - 1 and m.partial_candidates == {a}
    assert t.match([5]).num_tokens == 0


def test_grow_rekeys_in_place():
    t = PageTree(B)
    a = t.publish(t.root, 1, FULL)
    c = t.publish(a, 2, [1, 2, 3])
    assert t.grow(c, [1, 2, 3, 4, 5]) is c
    assert c.tokens == (1, 2, 3, 4, 5) and a.children == {(1, 2, 3, 4, 5): c}
    assert t.match(FULL + [1, 2, 3, 4, 5, 6]).pages == [a, c]


def test_grow_into_a_sibling_returns_the_sibling_and_changes_nothing():
    t = PageTree(B)
    a = t.publish(t.root, 1, FULL)
    c = t.publish(a, 2, [1, 2, 3])
    d = t.publish(a, 3, list(range(1, 9)))
    assert t.grow(c, list(range(1, 9))) is d
    assert c.tokens == (1, 2, 3) and a.children[(1, 2, 3)] is c


def test_grow_must_strictly_extend():
    t = PageTree(B)
    c = t.publish(t.root, 1, [1, 2, 3])
    with pytest.raises(AssertionError):
        t.grow(c, [1, 2, 3])
    with pytest.raises(AssertionError):
        t.grow(c, [1, 2, 4, 5])


def test_evict_takes_leaves_only_and_keeps_shared_trie_paths():
    t = PageTree(B)
    a = t.publish(t.root, 1, FULL)
    c = t.publish(a, 2, [1, 2, 3, 4, 5])
    d = t.publish(a, 3, list(range(1, 9)))
    with pytest.raises(AssertionError):
        t.evict(a)
    assert t.evict(c) == 2 and 2 not in t.nodes
    m = t.match(FULL + [1, 2, 3, 4, 5, 77])
    assert m.pages == [a] and m.partial_len == 5 and m.partial_candidates == {d}
    assert t.evict(d) == 3 and not a.children and not a.trie.root.next
    assert t.evict(a) == 1
    assert not t.root.children and not t.root.trie.root.next and not t.nodes

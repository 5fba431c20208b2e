"""Token trie and prefix index on their own, with the cases the reference's tests pin for its
page tree (tests/test_page_tree.py:12-120, page size 8), restated for an index that names pages by
their ids and has no table of children beside the trie."""

import pytest

from tinyserve_llm_amd.cache.prefix_index import TOP, PrefixIndex
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
            if run not in runs.values():                   # (two pages never hold the same run: the index swaps to the first)
                runs[page] = run
                trie.insert(page, run), plain.insert(page, run)
        elif what < 0.55:
            page = rng.choice(list(runs))
            longer = runs[page] + [rng.randrange(3) for _ in range(rng.randint(1, 4))]
            if longer not in runs.values():
                runs[page] = longer
                trie.insert(page, longer), plain.insert(page, longer)
        elif what < 0.8:
            page = rng.choice(list(runs))
            run = runs.pop(page)
            trie.remove(page, run), plain.remove(page, run)
        probe = tuple(rng.randrange(3) for _ in range(rng.randint(0, 12)))
        assert trie.longest_match(probe) == plain.longest_match(probe), f"step {step}: {probe}"
        assert trie.exact(probe) is next((page for page, run in runs.items() if tuple(run) == probe), None)
        for page, run in runs.items():
            depth, pages = trie.longest_match(run)
            assert depth == len(run) and page in pages and trie.exact(run) is page
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


def test_the_trie_marks_where_a_run_ends():
    trie, p, q = TokenTrie(), "p", "q"
    trie.insert(p, [1, 2, 3])
    trie.insert(q, [1, 2])
    assert trie.exact([1, 2]) == q and trie.exact([1, 2, 3]) == p and trie.exact([1]) is None
    assert trie.find((1, 2, 7)) == (2, {p, q}, q)
    trie.insert(q, [1, 2, 5, 6])                       # q's run gets longer: its old end is no end any more
    assert trie.exact([1, 2]) is None and trie.exact([1, 2, 5, 6]) == q
    trie.remove(p, [1, 2, 3])
    assert trie.exact([1, 2, 3]) is None and trie.find((1, 2, 3)) == (2, {q}, None)


def test_add_returns_the_page_that_was_there_on_a_duplicate():
    t = PrefixIndex(B)
    assert t.add(TOP, 1, FULL) == 1 and list(t) == [1] and t.tokens(1) == tuple(FULL)
    assert t.add(TOP, 2, FULL) == 1 and 2 not in t


def test_add_needs_a_full_page_before_it_and_a_new_page():
    t = PrefixIndex(B)
    t.add(TOP, 1, [7, 7])
    with pytest.raises(AssertionError):
        t.add(1, 2, [1])
    t.add(TOP, 3, FULL)
    with pytest.raises(AssertionError):
        t.add(3, 3, [1])
    with pytest.raises(AssertionError):
        t.add(3, 4, [])


def test_lookup_walks_full_pages_and_takes_over_a_page_that_holds_exactly_the_rest():
    t = PrefixIndex(B)
    t.add(TOP, 1, FULL)
    t.add(1, 2, [1, 2, 3])
    hit = t.lookup(FULL + [1, 2, 3, 99])
    assert hit.pages == [1, 2] and hit.tail == 0 and hit.num_tokens == 11


def test_lookup_reports_a_shared_beginning_with_the_pages_that_hold_it():
    t = PrefixIndex(B)
    t.add(TOP, 1, FULL)
    t.add(1, 2, [1, 2, 3])
    hit = t.lookup(FULL + [1, 2, 9, 9])
    assert hit.pages == [1] and hit.tail == 2 and hit.tail_holders == {2} and hit.num_tokens == 10


def test_lookup_never_covers_the_last_token():
    t = PrefixIndex(B)
    t.add(TOP, 1, FULL)
    hit = t.lookup(FULL)
    assert hit.pages == [] and hit.tail == B - 1 and hit.tail_holders == {1}
    assert t.lookup([5]).num_tokens == 0 and t.lookup([]).num_tokens == 0


def test_extend_keeps_the_page_findable_under_its_longer_run():
    t = PrefixIndex(B)
    t.add(TOP, 1, FULL)
    t.add(1, 2, [1, 2, 3])
    assert t.extend(2, [1, 2, 3, 4, 5]) == 2
    assert t.tokens(2) == (1, 2, 3, 4, 5) and not t.is_leaf(1) and t.is_leaf(2)
    assert t.lookup(FULL + [1, 2, 3, 4, 5, 6]).pages == [1, 2]
    short = t.lookup(FULL + [1, 2, 3, 6])
    assert short.pages == [1] and short.tail == 3 and short.tail_holders == {2}, "no page holds just the old run any more"


def test_extend_into_a_neighbour_returns_the_neighbour_and_changes_nothing():
    t = PrefixIndex(B)
    t.add(TOP, 1, FULL)
    t.add(1, 2, [1, 2, 3])
    t.add(1, 3, list(range(1, 9)))
    assert t.extend(2, list(range(1, 9))) == 3
    assert t.tokens(2) == (1, 2, 3) and t.lookup(FULL + [1, 2, 3, 0]).pages == [1, 2]


def test_extend_goes_on_after_the_pages_own_tokens():
    t = PrefixIndex(B)
    t.add(TOP, 1, [1, 2, 3])
    with pytest.raises(AssertionError):
        t.extend(1, [1, 2, 3])
    with pytest.raises(AssertionError):
        t.extend(1, [1, 2, 4, 5])


def test_discard_takes_pages_that_nothing_follows_and_keeps_shared_paths():
    t = PrefixIndex(B)
    t.add(TOP, 1, FULL)
    t.add(1, 2, [1, 2, 3, 4, 5])
    t.add(1, 3, list(range(1, 9)))
    with pytest.raises(AssertionError):
        t.discard(1)
    t.discard(2)
    assert 2 not in t
    hit = t.lookup(FULL + [1, 2, 3, 4, 5, 77])
    assert hit.pages == [1] and hit.tail == 5 and hit.tail_holders == {3}
    t.discard(3)
    assert t.is_leaf(1) and t.lookup(FULL + [1, 2]).num_tokens == B
    t.discard(1)
    assert len(t) == 0 and t.lookup(FULL + [1]).num_tokens == 0

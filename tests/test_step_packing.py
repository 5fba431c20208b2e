"""The step's integer layout, on the CPU: the general packing and the decode-only packing agree."""

import random
from types import SimpleNamespace

import pytest

from tinyserve_llm_amd.engine.runner import DecodeGraphs, ModelRunner, StepEntry, StepError


class View:
    def __init__(self, tables, slots):
        self.tables, self.slots = tables, slots

    def block_table(self, seq_id, space=0):
        return self.tables[space][seq_id]

    def state_slot(self, seq_id):
        return self.slots[seq_id]


def runner(page_size, pages, windows, tables, slots, vocab=100, max_pos=4096):
    r = ModelRunner.__new__(ModelRunner)
    r.storage = SimpleNamespace(page_size=page_size, spaces=[SimpleNamespace(num_pages=n, window=w) for n, w in zip(pages, windows)])
    r.model = SimpleNamespace(spec=SimpleNamespace(vocab_size=vocab, max_position=max_pos))
    r.view = View(tables, slots)
    r.windows = list(windows)
    return r


@pytest.mark.parametrize("windows", [(0,), (0, 40)])
def test_decode_packing_equals_general_packing(windows):
    rng = random.Random(5)
    ps, pages = 16, [64] * len(windows)
    for _ in range(30):
        n = rng.randrange(1, 7)
        starts = [rng.randrange(0, 200) for _ in range(n)]
        tables = []
        for sp, w in enumerate(windows):
            per = {}
            for i, st in enumerate(starts):
                t = [rng.randrange(pages[sp]) for _ in range(st // ps + 1 + rng.randrange(2))]
                if w:
                    for j in range(max(0, (st - w + 1) // ps)):     # pages the window has passed
                        t[j] = -1
                per[10 + i] = t
            tables.append(per)
        slots = {10 + i: rng.randrange(8) for i in range(n)}
        r = runner(ps, pages, windows, tables, slots)
        entries = [StepEntry(10 + i, [rng.randrange(100)], st, [0]) for i, st in enumerate(starts)]
        width = max(len(t) for per in tables for t in per.values()) + 1
        size = n + rng.randrange(3)
        a = r._pack(entries, [width] * len(windows), pad_to=size)
        b = r._pack_decode(entries, [width] * len(windows), pad_to=size)
        assert a[0] == b[0] and a[1] == b[1] and a[2] == b[2]


def test_general_packing_lays_out_portions_of_prompts():
    """Tokens, positions, request of each token, lengths, wanted rows, padded block tables and the
    cache slot of every token (page * page size + place in the page), for portions that start
    inside a page, cross pages and end at a page's edge, beside a single decoded token."""
    ps = 8
    tables = [{1: [5, 2, 9], 2: [7, 0, 3, 6], 3: [4]}]
    r = runner(ps, [16], (0,), tables, {1: 2, 2: 0, 3: 1})
    entries = [StepEntry(1, list(range(20, 31)), 6, [10]),        # positions 6..16: three pages
               StepEntry(2, [50], 25, [0]),                       # one decoded token, fourth page
               StepEntry(3, list(range(60, 68)), 0, [0, 7])]      # a whole page, to its edge
    flat, (T, S, R, widths, offsets, slot_offset), host = r._pack(entries)
    assert (T, S, R, widths) == (20, 3, 4, [4])
    ids = list(range(20, 31)) + [50] + list(range(60, 68))
    positions = list(range(6, 17)) + [25] + list(range(8))
    seq_of = [0] * 11 + [1] + [2] * 8
    assert flat[:T] == ids and flat[T:2 * T] == positions and flat[2 * T:3 * T] == seq_of
    assert flat[3 * T:3 * T + 4] == [0, 11, 12, 20] == host["cu"]
    assert flat[3 * T + 4:3 * T + 7] == [17, 26, 8] == host["ctx_lens"]
    assert flat[3 * T + 7:3 * T + 10] == [2, 0, 1]
    assert flat[3 * T + 10:3 * T + 14] == [10, 11, 12, 19]
    assert flat[offsets[0]:offsets[0] + 12] == [5, 2, 9, 0, 7, 0, 3, 6, 4, 0, 0, 0]
    table_of = {0: tables[0][1], 1: tables[0][2], 2: tables[0][3]}
    want = [table_of[s][p // ps] * ps + p % ps for s, p in zip(seq_of, positions)]
    assert flat[slot_offset:slot_offset + T] == want and len(flat) == slot_offset + T


def test_decode_packing_refuses_what_the_general_packing_refuses():
    r = runner(16, [8], (0,), [{1: [3, 9]}], {1: 0})
    for bad in ([StepEntry(1, [100], 5, [0])], [StepEntry(1, [5], 40, [0])], [StepEntry(1, [5], 20, [0])],
                [StepEntry(1, [5], 5, [0]), StepEntry(1, [6], 6, [0])]):
        with pytest.raises(StepError):
            r._pack_decode(bad, [4], pad_to=0)
        with pytest.raises((StepError, IndexError)):
            r._pack(bad, [4], pad_to=0)


def test_draw_words_round_trip():
    import torch
    words, start = DecodeGraphs._with_draws([1, 2, 3], 4, ([0.5, 0.0, 1.25], [5, (1 << 63) - 1, 0x123456789ABCDEF]))
    assert start == 4 and words.dtype == torch.int32 and len(words) == 4 + 4 * 4
    assert words[start:start + 8].view(torch.int64).tolist() == [5, (1 << 63) - 1, 0x123456789ABCDEF, 0]
    assert words[start + 8:start + 12].view(torch.float32).tolist() == [0.5, 0.0, 1.25, 0.0]
    assert words[start + 12:].tolist() == [-1] * 4, "no entry takes its token from the step before"
    fed, _ = DecodeGraphs._with_draws([1, 2, 3], 4, ([0.5, 0.0, 1.25], [5, 6, 7]), feed=[2, -1, 0])
    assert fed[start + 12:].tolist() == [2, -1, 0, -1], "the rows of the step before, then the idle rows"
    none, _ = DecodeGraphs._with_draws([1, 2], 2, None)
    assert none.tolist() == [1, 2, 0, 0, 0, 0, 0, 0, -1, -1]

"""Replay on the GPU against the plain implementation: the same requests whole, with the last 32
tokens decoded one by one, in portions of changing size, and mixed with other requests on so few
pages that pages are used again; in float32 and in bfloat16."""

from __future__ import annotations

import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from tests.helpers import CONFIGS, make_folder, prompt
from tests.plain.llama import PlainLlama

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LENGTHS = {"A": [5, 17, 33, 100], "B": [1, 40, 70, 129]}

# float32 engine against the float64 oracle: only the engine's own 32-bit rounding separates them.
# bfloat16 engine against the float64 oracle on bfloat16-rounded weights: activations are rounded
# to 8 bits of mantissa a few dozen times on the way to a logit. The worst logit is off by 2.6e-3 to
# 4.9e-3 in every way of feeding (the logits' spread is 0.16); the bound is twice that.
TOL = {"float32": dict(atol=5e-6, rtol=1e-5), "bfloat16": dict(atol=1e-2, rtol=0.0)}


@pytest.fixture(scope="module", params=["A", "B"])
def case(request, tmp_path_factory):
    name = request.param
    folder = make_folder(tmp_path_factory, name)
    config = CONFIGS[name][0]
    prompts = [prompt(100 + i, n, config.vocab_size) for i, n in enumerate(LENGTHS[name])]
    oracles = {}
    for dtype, stored in (("float32", None), ("bfloat16", torch.bfloat16)):
        plain = PlainLlama(folder, torch.float64, weights_as=stored)
        oracles[dtype] = [plain.logits(p) for p in prompts]
    return name, folder, config, prompts, oracles


def replayer(folder, dtype, max_tokens):
    from tinyserve_llm_amd.engine.replay import Replay
    return Replay(folder, dtype, max_tokens)


def check(got: dict[tuple[int, int], torch.Tensor], oracle, dtype: str):
    """got maps (request, position) to a logits row."""
    assert got, "nothing was compared"
    worst = 0.0
    for (r, pos), row in got.items():
        want = oracle[r][pos]
        torch.testing.assert_close(row.double().cpu(), want, **TOL[dtype], msg=lambda m: f"request {r} position {pos}: {m}")
        worst = max(worst, float((row.double().cpu() - want).abs().max()))
    print(f"[{dtype}] worst absolute logit error {worst:.3e} over {len(got)} rows")
    return worst


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_requests_alone(case, dtype):
    name, folder, config, prompts, oracles = case
    rep = replayer(folder, dtype, 256)
    got = {}
    for r, p in enumerate(prompts):
        logits = rep.step([{"id": f"r{r}", "tokens": p, "want": list(range(len(p)))}], [f"r{r}"])
        assert logits.shape == (len(p), config.vocab_size) and logits.dtype == torch.float32
        for pos in range(len(p)):
            got[(r, pos)] = logits[pos]
    check(got, oracles[dtype], dtype)
    assert rep.manager.num_available_blocks() == rep.manager.num_blocks, "every page came back"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_last_32_tokens_one_by_one(case, dtype):
    name, folder, config, prompts, oracles = case
    rep = replayer(folder, dtype, 256)
    got = {}
    for r, p in enumerate(prompts):
        head = max(0, len(p) - 32)
        if head:
            logits = rep.step([{"id": f"r{r}", "tokens": p[:head], "want": [head - 1]}], [])
            got[(r, head - 1)] = logits[0]
        for pos in range(head, len(p)):
            logits = rep.step([{"id": f"r{r}", "tokens": [p[pos]], "want": [0]}], [f"r{r}"] if pos == len(p) - 1 else [])
            got[(r, pos)] = logits[0]
    check(got, oracles[dtype], dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_portions_of_changing_size(case, dtype):
    name, folder, config, prompts, oracles = case
    rep = replayer(folder, dtype, 256)
    sizes = [2, 7, 3, 16, 2, 5, 31, 2, 64, 9]
    got = {}
    for r, p in enumerate(prompts):
        pos, i = 0, r
        while pos < len(p):
            n = min(sizes[i % len(sizes)], len(p) - pos)
            i += 1
            want = sorted({0, n - 1})
            logits = rep.step([{"id": f"r{r}", "tokens": p[pos:pos + n], "want": want}],
                              [f"r{r}"] if pos + n == len(p) else [])
            for j, w in enumerate(want):
                got[(r, pos + w)] = logits[j]
            pos += n
    check(got, oracles[dtype], dtype)


MIXED_LENGTHS = {"A": [100, 33, 17, 5, 70, 120, 64, 9], "B": [129, 70, 40, 1, 65, 100, 128, 30, 200]}


def mixed_schedule(prompts, pool_pages, page=64, most_live=4):
    """Steps that keep up to four requests live on `pool_pages` pages: requests start in the order
    given as soon as the pages for their whole length are free, feed portions of changing size
    (often a single token) and end at different times, so that a request that starts later gets the
    pages of one that has ended while others are still in the middle of theirs. Returns a list of
    (entries, end) with entries (request, start, count, want)."""
    cursors = [0] * len(prompts)
    pages = [-(-len(p) // page) for p in prompts]
    chunk = [13, 2, 1, 7, 1, 1, 30, 1, 3, 1]
    waiting, live, steps, tick = list(range(len(prompts))), [], [], 0
    while waiting or live:
        while waiting and len(live) < most_live and sum(pages[r] for r in live) + pages[waiting[0]] <= pool_pages:
            live.append(waiting.pop(0))
        entries, end = [], []
        for k, r in enumerate(live):
            n = min(len(prompts[r]) - cursors[r], chunk[(tick + 3 * r) % len(chunk)])
            entries.append((r, cursors[r], n, [n - 1] if n > 1 else [0]))
            cursors[r] += n
            if cursors[r] == len(prompts[r]):
                end.append(r)
        live = [r for r in live if r not in end]
        steps.append((entries, end))
        tick += 1
    return steps


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mixed_requests_on_few_pages(case, dtype):
    """Eight or nine different requests on a pool that holds the first four (each rounded up to pages of
    64): the later ones run on pages that earlier ones have written and given back, while other
    requests are in the middle of theirs. A stale page holds another request's keys, so a write
    that was skipped, or a page number that went to the wrong request, shows in the logits."""
    name, folder, config, _, _ = case
    prompts = [prompt(300 + i, n, config.vocab_size) for i, n in enumerate(MIXED_LENGTHS[name])]
    plain = PlainLlama(folder, torch.float64, weights_as=torch.bfloat16 if dtype == "bfloat16" else None)
    oracle = [plain.logits(p) for p in prompts]
    pool = sum(-(-len(p) // 64) for p in prompts[:4])
    rep = replayer(folder, dtype, 64 * pool)
    assert rep.manager.num_blocks == pool
    got, given_back, taken_again_beside = {}, set(), 0
    for entries, end in mixed_schedule(prompts, pool):
        batch = [{"id": f"q{r}", "tokens": prompts[r][s:s + n], "want": w} for r, s, n, w in entries]
        held = {r: set(rep.manager.block_table(rep.ids[f"q{r}"])) for r, s, _, _ in entries if s}
        logits = rep.step(batch, [])
        for r, s, n, w in entries:
            if s == 0 and set(rep.manager.block_table(rep.ids[f"q{r}"])) & given_back and len(held) >= 2:
                taken_again_beside += 1
        row = 0
        for r, s, n, w in entries:
            for j in w:
                got[(r, s + j)] = logits[row]
                row += 1
        assert row == logits.shape[0]
        for r in end:
            given_back |= set(rep.manager.block_table(rep.ids[f"q{r}"]))
        rep.step([], [f"q{r}" for r in end])
    assert taken_again_beside >= 2, "requests started on used pages while two others were live"
    check(got, oracle, dtype)
    assert rep.manager.num_available_blocks() == rep.manager.num_blocks


def test_bfloat16_logits_of_one_token_at_a_time_stay_with_those_of_the_whole_prompt(case):
    """In bfloat16 a step of up to 16 rows applies the norm inside the projection kernels (the operand
    is (x + residual) * weight rounded once, the row's scale multiplies the finished sums), a larger
    step runs the norm as a kernel of its own (rounded before the weight, as the reference does), and
    attention takes the split-key kernel or the tile kernel: the same request fed whole and fed token
    by token goes through different roundings at every layer. Both are held to the plain model
    elsewhere; here they are held to each other, at the last 32 positions, where token-by-token
    feeding has gone through its own roundings the longest."""
    name, folder, config, prompts, oracles = case
    worst = 0.0
    for r, p in enumerate(prompts):
        if len(p) < 40:
            continue
        rep = replayer(folder, "bfloat16", 512)
        tail = list(range(len(p) - 32, len(p)))
        whole = rep.step([{"id": "w", "tokens": p, "want": tail}], ["w"])
        rep.step([{"id": "s", "tokens": p[:len(p) - 32], "want": []}], [])
        single = torch.cat([rep.step([{"id": "s", "tokens": [p[pos]], "want": [0]}], []) for pos in tail])
        diff = float((whole - single).abs().max())
        worst = max(worst, diff)
        assert diff <= TOL["bfloat16"]["atol"], f"request {r}: fed whole and fed singly differ by {diff:.3e}"
        for got in (whole, single):       # and neither has drifted from the plain model
            torch.testing.assert_close(got.double().cpu(), oracles["bfloat16"][r][tail[0]:], **TOL["bfloat16"])
    print(f"worst difference between the two ways of feeding: {worst:.3e}")
    if name == "B":      # (configuration A's head size of 16 goes to the one kernel that serves every step alike)
        assert worst > 0.0, "the two ways take different attention kernels; equal results would mean one of them did not run"


def test_float32_logits_do_not_depend_on_the_cut(case):
    """In float32 every kernel fixes the order of its sums per row, so logits are bit-equal
    however the tokens were cut into steps and whatever else was in the batch."""
    name, folder, config, prompts, oracles = case
    rep = replayer(folder, "float32", 512)
    p = prompts[-1]
    whole = rep.step([{"id": "w", "tokens": p, "want": list(range(len(p)))}], ["w"])
    other = prompts[-2]
    pos, got = 0, []
    rep.step([{"id": "o", "tokens": other[:3], "want": []}], [])
    for n in [1, 2, 9, 1, 30, 64, 2, 1000]:
        n = min(n, len(p) - pos)
        if n == 0:
            break
        batch = [{"id": "c", "tokens": p[pos:pos + n], "want": list(range(n))}]
        if pos % 2:
            batch.insert(0, {"id": "o", "tokens": [other[3 + pos % 5]], "want": [0]})
        logits = rep.step(batch, [])
        got.append(logits[-n:])
        pos += n
    assert torch.equal(torch.cat(got), whole)


def test_trace_run_program(case, tmp_path):
    """bin/trace_run as a user runs it: JSON lines in, `done <step>` lines and .f32 files out."""
    name, folder, config, prompts, oracles = case
    p = prompts[2]
    lines = [
        {"step": 0, "entries": [{"id": "a", "tokens": p[:10], "want": [0, 9]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": p[10:12], "want": []}], "end": []},
        {"step": 2, "entries": [{"id": "a", "tokens": p[12:], "want": [len(p) - 13]},
                                {"id": "b", "tokens": prompts[1], "want": [len(prompts[1]) - 1]}], "end": ["a", "b"]},
    ]
    out = tmp_path / "out"
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "float32",
                        "--out", str(out), "--max-tokens", str(-(-len(p) // 64) * 64 + -(-len(prompts[1]) // 64) * 64)],
                       input="\n".join(json.dumps(x) for x in lines) + "\n", capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr
    assert r.stdout.split() == ["done", "0", "done", "1", "done", "2"]
    assert not (out / "1.f32").exists()
    s0 = np.fromfile(out / "0.f32", dtype="<f4").reshape(2, config.vocab_size)
    s2 = np.fromfile(out / "2.f32", dtype="<f4").reshape(2, config.vocab_size)
    got = {(2, 0): torch.from_numpy(s0[0]), (2, 9): torch.from_numpy(s0[1]),
           (2, len(p) - 1): torch.from_numpy(s2[0]), (1, len(prompts[1]) - 1): torch.from_numpy(s2[1])}
    check(got, oracles["float32"], "float32")


def drawn_configuration(rng):
    """A configuration whose every size is drawn: head sizes in steps of 16 up to 256, any grouping, widths and
    vocabularies that are no power of two (down to a width of 2 and a vocabulary of 2)."""
    from tinyserve_llm_amd.config import LlamaConfig, RopeScaling
    kv = rng.choice([1, 1, 2, 3, 4, 8])
    scaling = None
    if rng.random() < 0.5:
        scaling = RopeScaling(factor=rng.choice([2.0, 8.0, 32.0]), low_freq_factor=1.0, high_freq_factor=rng.choice([2.0, 4.0]),
                              original_max_position_embeddings=rng.choice([16, 64, 128]))
    vocab = rng.choice([2, 17, 100, 255, 256, 333, 1001, 4099])
    return LlamaConfig(
        vocab_size=vocab, hidden_size=rng.choice([2, 10, 40, 64, 100, 136, 258, 520, 1024]),
        intermediate_size=rng.choice([2, 30, 100, 128, 150, 300, 520, 1026]), num_hidden_layers=rng.choice([1, 2, 3]),
        num_attention_heads=kv * rng.choice([1, 1, 2, 3, 4, 5, 7, 8]), num_key_value_heads=kv,
        head_dim=rng.choice([16, 32, 48, 64, 80, 96, 112, 128, 160, 192, 256]), max_position_embeddings=512,
        rms_norm_eps=rng.choice([1e-5, 1e-6, 1e-3]), rope_theta=rng.choice([10000.0, 500000.0]), rope_scaling=scaling,
        tie_word_embeddings=rng.random() < 0.5, eos_token_id=vocab - 1)


def drawn_schedule(rng, prompts, pool_pages, page=64, most_live=4):
    """Steps as in `mixed_schedule`, with everything drawn: the portions (one way of cutting a case: whole prompts,
    all but the last 32 tokens and then single ones, portions of one to three tokens, or anything up to 100), the
    places whose logits are wanted (none, some, not always the last) and requests left out of a step."""
    cursors = [0] * len(prompts)
    pages = [-(-len(p) // page) for p in prompts]
    waiting, live, steps = list(range(len(prompts))), [], []
    way = rng.choice(["whole", "tail", "tiny", "any"])
    while waiting or live:
        while waiting and len(live) < most_live and sum(pages[r] for r in live) + pages[waiting[0]] <= pool_pages:
            live.append(waiting.pop(0))
        entries, end = [], []
        for r in live:
            if len(live) > 1 and rng.random() < 0.15:
                continue
            left = len(prompts[r]) - cursors[r]
            n = {"whole": left, "tail": left - 32 if left > 32 else 1, "tiny": rng.choice([1, 2, 2, 3]),
                 "any": rng.choice([1, 1, 1, 2, 3, 7, 13, 16, 17, 31, 32, 33, 64, 65, 100])}[way]
            n = max(1, min(n, left))
            want = sorted(set(rng.sample(range(n), min(n, rng.choice([0, 1, 1, 2, 3]))) + ([n - 1] if rng.random() < 0.7 else [])))
            entries.append((r, cursors[r], n, want))
            cursors[r] += n
            if cursors[r] == len(prompts[r]):
                end.append(r)
        live = [r for r in live if r not in end]
        if entries:
            steps.append((entries, end))
    return steps


@pytest.mark.parametrize("seed", range(24))
def test_drawn_configurations_and_schedules(seed, tmp_path):
    """Neither the sizes nor the schedule are this file's choice: a configuration, two to seven prompts of 1 to 300
    tokens, a pool that holds the four longest, and a schedule are drawn per case, and both precisions are compared
    with the plain model at every wanted place. The bounds are relative to the logits' spread: 2e-5 of it in
    float32 (1.6e-6 is the worst of 7,500 such cases), 4 % in bfloat16 (0.62 % is)."""
    import random

    from tinyserve_llm_amd.weights.random_init import write_random_model
    rng = random.Random(50000 + seed)
    config = drawn_configuration(rng)
    lengths = [rng.choice([1, 2, 5, 17, 33, 63, 64, 65, 100, 128, 129, 200, 257, 300]) for _ in range(rng.randint(2, 7))]
    prompts = [[rng.randrange(config.vocab_size) for _ in range(n)] for n in lengths]
    write_random_model(str(tmp_path), config, seed, rng.choice([torch.float32, torch.bfloat16]))
    pool = sum(sorted((-(-n // 64) for n in lengths), reverse=True)[:4])
    steps = drawn_schedule(rng, prompts, pool)
    for dtype, bound in (("float32", 2e-5), ("bfloat16", 4e-2)):
        plain = PlainLlama(str(tmp_path), torch.float64, weights_as=torch.bfloat16 if dtype == "bfloat16" else None)
        oracle = [plain.logits(p) for p in prompts]
        spread = max(float(o.max() - o.min()) for o in oracle)
        rep = replayer(str(tmp_path), dtype, 64 * pool)
        compared = 0
        for entries, end in steps:
            logits = rep.step([{"id": f"q{r}", "tokens": prompts[r][s:s + n], "want": w} for r, s, n, w in entries],
                              [f"q{r}" for r in end])
            assert logits.shape[0] == sum(len(w) for _, _, _, w in entries)
            row = 0
            for r, s, n, w in entries:
                for j in w:
                    off = float((logits[row].double().cpu() - oracle[r][s + j]).abs().max())
                    assert off <= bound * spread, f"{dtype}, request {r}, position {s + j}: off by {off:.3e} of a spread of {spread:.3e}"
                    row += 1
                    compared += 1
        assert rep.manager.num_available_blocks() == rep.manager.num_blocks, "every page came back"
        print(f"[{dtype}] {compared} rows compared")

"""Generation through the entry point on the GPU: greedy tokens against the plain
implementation; nothing the cache or the scheduler does (prefix hits, portions, preemption,
forks, caching off) may change what is generated; long decoding; the first tokens of a sequence."""

from __future__ import annotations

import json
import os
import subprocess
import sys

import pytest
import torch

from tests.helpers import CONFIGS, make_folder, prompt
from tests.plain.llama import PlainLlama

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def folder_a(tmp_path_factory):
    return make_folder(tmp_path_factory, "A")


@pytest.fixture(scope="module")
def folder_b(tmp_path_factory):
    return make_folder(tmp_path_factory, "B")


def engine(folder, dtype=torch.float32, num_blocks=64, block_size=4, caching=True, seed=None, **over):
    from tinyserve_llm_amd.engine.llm import LLM, CacheConfig
    from tinyserve_llm_amd.engine.scheduler import SchedulerConfig
    sc = SchedulerConfig(**{**dict(max_model_len=96, max_num_seqs=8, max_num_batched_tokens=104), **over})
    return LLM(folder, sc, CacheConfig(block_size=block_size, caching=caching), dtype=dtype, num_blocks=num_blocks,
               seed=seed)


def greedy(max_tokens=12, **kw):
    from tinyserve_llm_amd.engine.sequence import SamplingParams
    return SamplingParams(max_tokens=max_tokens, temperature=0.0, ignore_eos=True, **kw)


PREFIX = [5, 17, 3, 99, 42, 8, 61, 23, 7]     # two full pages of 4 and a partial one
PROMPTS = [PREFIX + [11, 12], PREFIX + [30], [77, 2, 9], PREFIX + [11, 12, 13, 14, 15], [64] * 6]


def test_greedy_equals_the_plain_implementation_and_prefixes_are_reused(folder_a):
    """tests/test_engine.py:142-154 of the reference, against our own oracle."""
    plain = PlainLlama(folder_a, torch.float64)
    llm = engine(folder_a)
    results = llm.generate(PROMPTS, greedy())
    for p, r in zip(PROMPTS, results):
        assert r.token_ids == [plain.greedy(p, 12)] and r.finish_reasons == ["length"]
        assert r.prompt_token_ids == p and r.texts is None
    assert llm.scheduler.stats().cached_tokens == 0, "all admitted in one step, nothing was committed yet"
    later = PREFIX + [11, 40]
    (r,) = llm.generate([later], greedy())
    assert r.token_ids == [plain.greedy(later, 12)]
    assert llm.scheduler.stats().cached_tokens == len(PREFIX) + 1, "the released prefix pages were found again"
    assert llm.manager.stats().blocks_in_use == 0


@pytest.mark.parametrize("caching", [True, False])
def test_preemption_portions_and_caching_do_not_change_the_output(folder_a, caching):
    """tests/test_engine.py:157-166: a pool too small for all five forces preemption."""
    expected = [r.token_ids for r in engine(folder_a).generate(PROMPTS, greedy())]
    small = engine(folder_a, num_blocks=14, caching=caching)
    assert [r.token_ids for r in small.generate(PROMPTS, greedy())] == expected
    st = small.scheduler.stats()
    assert st.preemptions > 0 and (st.cached_tokens > 0) == caching
    cut = engine(folder_a, caching=caching, max_num_batched_tokens=9, max_prefill_chunk=3)
    assert [r.token_ids for r in cut.generate(PROMPTS, greedy())] == expected
    assert max(s.num_tokens for s in cut.steps) <= 9
    first = engine(folder_a, caching=caching, step_mode="prefill_first", max_prefill_chunk=5)
    assert [r.token_ids for r in first.generate(PROMPTS, greedy())] == expected


def test_parallel_samples_fork_and_greedy_samples_agree(folder_b):
    plain = PlainLlama(folder_b, torch.float64)
    llm = engine(folder_b)
    p = prompt(1, 13, 384)
    (r,) = llm.generate([p], greedy(6, n=3))
    assert r.token_ids == [plain.greedy(p, 6)] * 3
    st = llm.manager.stats()
    assert st.blocks_in_use == 0 and st.cow_copies >= 2, "the shared tail page was copied by the writers"


def test_sampling_is_seeded_and_does_not_depend_on_the_batch(folder_b):
    from tinyserve_llm_amd.engine.sequence import SamplingParams
    sp = SamplingParams(max_tokens=10, temperature=0.7, n=2, ignore_eos=True)
    prompts = [prompt(i, n, 384) for i, n in enumerate((1, 40, 70, 29))]
    a = [r.token_ids for r in engine(folder_b, seed=3).generate(prompts, sp)]
    b = [r.token_ids for r in engine(folder_b, seed=3).generate(prompts, sp)]
    c = [r.token_ids for r in engine(folder_b, seed=4).generate(prompts, sp)]
    assert a == b and a != c
    assert all(x[0] != x[1] for x in a), "the two samples of a request draw different noise"
    # the same requests in portions, on a pool that forces preemption: same draws, since the
    # noise is keyed by (request, sample, output position) and float32 logits do not depend on the cut
    d = [r.token_ids for r in engine(folder_b, seed=3, num_blocks=50, max_num_batched_tokens=24,
                                     max_prefill_chunk=16).generate(prompts, sp)]
    assert d == a


def race_scores(plain_row, temperature, seed, request, sample, position):
    """What the sampler maximises, from the plain model's logits and the kernel's noise written out
    on the host: logit / t - log E(seed, key of (request, sample, output position))."""
    from tests.test_gpu_kernels import exp_noise
    from tinyserve_llm_amd.sampling.sampler import row_key
    noise = exp_noise(seed, row_key(request, sample, position), plain_row.shape[0])
    return plain_row / temperature - noise.log()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shared", [64, 75])
def test_drawn_tokens_of_a_workload_with_prefix_hits_forks_and_portions_against_the_plain_model(folder_b, dtype, shared):
    """Configuration B's workload as the baseline states it: prompts of 1, 40, 70 and 129 tokens, the
    last two behind a common prefix (64 tokens: two whole pages of 32; 75: it ends inside the third page,
    whose leading slots are copied), the second drawn twice (n = 2: the samples share the prompt's pages
    and copy its last one when they write), prompts fed in portions of 32 beside decoding requests,
    12 tokens each at temperature 0.7, prefix reuse on. The fourth arrives when the third has ended
    (only then is a page that is not full published), while the first two still decode. Every drawn
    token is checked against the plain model run whole on the same history: in float32 it is the one
    that wins the race under the kernel's noise; in bfloat16 it lies within a small gap of the winner."""
    from tinyserve_llm_amd.engine.sequence import SamplingParams
    vocab, seed, t = 384, 9, 0.7
    common = prompt(50, shared, vocab)
    tails = prompt(53, max(2, 70 - shared), vocab), prompt(54, 129 - shared, vocab)
    assert tails[0][0] != tails[1][0], "the prompts part right after the common prefix"
    prompts = [prompt(51, 1, vocab), prompt(52, 40, vocab), common + tails[0], common + tails[1]]
    lengths = [12, 12, 3, 12]
    plain = PlainLlama(folder_b, torch.float64, weights_as=torch.bfloat16)     # (the folder stores bfloat16 already)
    llm = engine(folder_b, dtype=dtype, block_size=32, num_blocks=24, seed=seed, max_model_len=160, max_num_seqs=8,
                 max_num_batched_tokens=48, max_prefill_chunk=32)

    def add(i):
        return llm.add_request(prompts[i], SamplingParams(max_tokens=lengths[i], temperature=t, n=2 if i == 1 else 1,
                                                          ignore_eos=True), arrival_time=float(i))

    ids = [add(0), add(1), add(2)]
    done = {}
    while llm.scheduler.has_unfinished():
        for out in llm.step():
            done[out.request_id] = out
        if ids[2] in done and len(ids) == 3:
            assert ids[0] not in done and ids[1] not in done, "the first two still decode when the fourth arrives"
            ids.append(add(3))
    st, cache = llm.scheduler.stats(), llm.manager.stats()
    assert st.cached_tokens == shared, "the fourth prompt found the third one's pages"
    assert cache.cow_copies >= 1, "the two samples copied the prompt's last page"
    assert cache.partial_copies == (1 if shared % 32 else 0)
    assert max(s.num_tokens for s in llm.steps) <= 48
    assert sum(s.num_seqs >= 4 and s.num_tokens >= 20 for s in llm.steps) >= 2, "portions ran beside decoding requests"
    checked = 0
    for rid, q, n in zip(ids, prompts, lengths):
        for seq in done[rid].sequences:
            history = list(q)
            assert len(seq.output_token_ids) == n
            for i, tok in enumerate(seq.output_token_ids):
                scores = race_scores(plain.logits(history)[-1], t, seed, rid, seq.sample_index, i)
                where = f"request {rid} sample {seq.sample_index} token {i}"
                if dtype == torch.float32:
                    top = torch.topk(scores, 2).values
                    assert tok == int(scores.argmax()) or float(top[0] - top[1]) < 1e-4, \
                        f"{where}: drew {tok}, the race's winner is {int(scores.argmax())}"
                else:
                    assert float(scores.max() - scores[tok]) <= 0.06, where
                history.append(tok)
                checked += 1
    assert checked == 12 + 2 * 12 + 3 + 12
    two = done[ids[1]].sequences
    assert two[0].output_token_ids != two[1].output_token_ids


def test_recording_a_step_while_a_dropped_engine_awaits_collection(folder_a):
    """An engine that holds recorded steps is dropped inside a reference cycle, so that only the
    collector can free it; a second engine then records its own steps with the collector set to run
    at every opportunity. The recording keeps the collector off (a graph destroyed inside a recording
    aborted the process once), and the second engine's tokens are the first one's."""
    import gc
    first = engine(folder_a)
    expected = [r.token_ids for r in first.generate(PROMPTS[:3], greedy(5))]
    assert first.runner.graphs.graphs, "the first engine holds recorded steps"
    first.myself = first
    gc.disable()                        # (the cycle stays pending while the second engine is built)
    old = gc.get_threshold()
    try:
        del first
        second = engine(folder_a)
        gc.set_threshold(1, 1, 1)
        gc.enable()
        got = [r.token_ids for r in second.generate(PROMPTS[:3], greedy(5))]
    finally:
        gc.set_threshold(*old)
        gc.enable()
    assert got == expected and second.runner.graphs.graphs


def test_the_end_token_stops_generation(folder_a):
    plain = PlainLlama(folder_a, torch.float64)
    full = plain.greedy(PROMPTS[0], 12)
    eos = full[2]
    llm = engine(folder_a, eos_token_id=eos)
    from tinyserve_llm_amd.engine.sequence import SamplingParams
    (r,) = llm.generate(PROMPTS[:1], SamplingParams(max_tokens=12, temperature=0.0))
    assert r.token_ids == [full[:full.index(eos) + 1]] and r.finish_reasons == ["eos"]


def test_step_records_requests_by_hand_and_timing(folder_a):
    llm = engine(folder_a)
    (r,) = llm.generate([PROMPTS[0]], greedy(3))
    assert [s.num_tokens for s in llm.steps] == [len(PROMPTS[0]), 1, 1] and all(s.start <= s.end for s in llm.steps)
    assert llm.steps[-1].scheduler.decode_tokens == 2 and llm.steps[-1].cache.publishes > 0
    assert r.arrival_time <= r.first_token_time <= r.finish_time
    rid = llm.add_request([1, 2, 3], greedy(2))
    outs = []
    while llm.scheduler.has_unfinished():
        outs += llm.step()
    assert [o.request_id for o in outs] == [rid]
    with pytest.raises(ValueError, match="vocabulary"):
        llm.add_request([1, 256], greedy(2))
    with pytest.raises(ValueError, match="tokenizer"):
        llm.add_request("text", greedy(2))
    with pytest.raises(ValueError, match="max_model_len"):
        llm.add_request([1] * 90, greedy(12))


def test_pool_sized_from_free_memory(folder_a):
    from tinyserve_llm_amd.engine.llm import LLM, CacheConfig
    from tinyserve_llm_amd.engine.scheduler import SchedulerConfig
    sc = SchedulerConfig(max_model_len=96, max_num_seqs=8, max_num_batched_tokens=104)
    llm = LLM(folder_a, sc, CacheConfig(block_size=16), dtype=torch.float32)
    assert llm.manager.num_blocks >= 8 * 7
    (r,) = llm.generate([PROMPTS[2]], greedy(4))
    assert len(r.token_ids[0]) == 4


@pytest.mark.parametrize("name", ["A", "B"])
def test_bfloat16_generation_stays_within_the_logit_gap(name, folder_a, folder_b):
    """In bfloat16 near-ties may flip a token, so tokens are judged by the oracle's logits: every
    generated token must be within a small gap of the oracle's best for the same history
    (the reference judges real-weight runs the same way, scripts/check_real_model.py:59-78)."""
    folder = folder_a if name == "A" else folder_b
    vocab = CONFIGS[name][0].vocab_size
    plain = PlainLlama(folder, torch.float64, weights_as=torch.bfloat16)
    llm = engine(folder, dtype=torch.bfloat16, block_size=16, num_blocks=32)
    prompts = [prompt(20 + i, n, vocab) for i, n in enumerate((5, 33, 60))]
    results = llm.generate(prompts, greedy(10))
    agree = total = 0
    for p, r in zip(prompts, results):
        ids = list(p)
        for tok in r.token_ids[0]:
            row = plain.logits(ids)[-1]
            assert float(row.max() - row[tok]) <= 0.03, "a token far from the oracle's best"
            agree += int(tok == int(row.argmax()))
            total += 1
            ids.append(tok)
    assert agree / total >= 0.8


def test_long_decoding_keeps_matching(folder_b):
    """150 tokens decoded one by one over five pages of 32: logits checked along the way."""
    from tinyserve_llm_amd.engine.replay import Replay
    ids = prompt(77, 200, 384)
    want = PlainLlama(folder_b, torch.float64).logits(ids)
    rep = Replay(folder_b, "float32", 256, page_size=32)
    rep.step([{"id": "x", "tokens": ids[:50], "want": []}], [])
    for pos in range(50, 200):
        row = rep.step([{"id": "x", "tokens": [ids[pos]], "want": [0]}], [])[0]
        if pos % 7 == 0 or pos in (63, 64, 95, 96, 127, 128, 199):
            torch.testing.assert_close(row.double().cpu(), want[pos], rtol=1e-5, atol=5e-6, msg=lambda m: f"position {pos}: {m}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens_of_a_sequence(folder_a, dtype):
    """Positions 0, 1, 2 fed one at a time: the first key alone, then two, then three."""
    from tinyserve_llm_amd.engine.replay import Replay
    ids = prompt(5, 4, 256)
    want = PlainLlama(folder_a, torch.float64, weights_as=torch.bfloat16 if dtype == "bfloat16" else None).logits(ids)
    rep = Replay(folder_a, dtype, 64)
    tol = dict(rtol=1e-5, atol=5e-6) if dtype == "float32" else dict(rtol=0.0, atol=1e-2)
    for pos in range(4):
        row = rep.step([{"id": "f", "tokens": [ids[pos]], "want": [0]}], [])[0]
        torch.testing.assert_close(row.double().cpu(), want[pos], **tol)


def test_command_line_writes_one_record(folder_a, tmp_path):
    out = tmp_path / "result.json"
    r = subprocess.run([sys.executable, "-m", "tinyserve_llm_amd.generate", "--model", folder_a, "--prompt-ids", "5,17,3",
                        "--prompt-ids", "77,2,9", "--max-tokens", "5", "--temperature", "0", "--ignore-eos", "--dtype",
                        "float32", "--block-size", "16", "--num-blocks", "16", "--max-model-len", "64", "--max-num-seqs", "4",
                        "--max-num-batched-tokens", "64", "--out", str(out)],
                       capture_output=True, text=True, cwd=ROOT, timeout=600)
    assert r.returncode == 0, r.stderr
    record = json.loads(out.read_text())
    plain = PlainLlama(folder_a, torch.float64)
    assert [c["token_ids"][0] for c in record["completions"]] == [plain.greedy([5, 17, 3], 5), plain.greedy([77, 2, 9], 5)]
    assert record["output_tokens"] == 10 and "wrote" in r.stdout


def test_decode_graphs_replay_what_eager_steps_compute(folder_b):
    """Decode steps come from HIP graphs (one per batch size, idle rows above eight requests);
    prompts and mixed steps run eagerly in between. Every replay must give what the eager engine
    gives: float32 logits are bit-equal, so the tokens are."""
    from tinyserve_llm_amd.engine.llm import LLM, CacheConfig
    from tinyserve_llm_amd.engine.scheduler import SchedulerConfig
    from tinyserve_llm_amd.engine.sequence import SamplingParams
    sc = SchedulerConfig(max_model_len=128, max_num_seqs=16, max_num_batched_tokens=80, max_prefill_chunk=32)
    prompts = [prompt(40 + i, 3 + 7 * i, 384) for i in range(13)]
    params = [SamplingParams(max_tokens=4 + 3 * (i % 5), temperature=0.8 if i % 2 else 0.0, ignore_eos=True) for i in range(13)]
    outs = []
    for graphs in (True, False):
        llm = LLM(folder_b, sc, CacheConfig(block_size=16), dtype=torch.float32, num_blocks=120, seed=5, decode_graphs=graphs)
        assert (llm.runner.graphs is not None) == graphs
        outs.append([r.token_ids for r in llm.generate(prompts, params)])
        if graphs:
            sizes = sorted({size for size, width in llm.runner.graphs.graphs})
            assert len(sizes) >= 3 and 16 in sizes, f"several batch sizes were captured, a padded one among them: {sizes}"
            again = [r.token_ids for r in llm.generate(prompts, params)]      # replays of graphs captured before
            # new request ids give new noise keys: only the greedy requests repeat exactly
            assert [a for a, p in zip(again, params) if not p.temperature] == \
                [a for a, p in zip(outs[0], params) if not p.temperature]
    assert outs[0] == outs[1]


@pytest.mark.parametrize("num_blocks", [120, 18])
def test_steps_closed_in_two_halves_generate_the_same(folder_b, num_blocks):
    """With `run_ahead` a decode step is scheduled, packed and started while the one before it
    still runs, from a placeholder for the token under way, which it takes on the device; a
    sequence that ends has a row in the step already started, which is dropped. Tokens must equal those of the engine that closes
    every step before it schedules the next: with sampling (keys name request, sample and position),
    with sequences that end by themselves, and with so few pages that sequences are preempted."""
    from tinyserve_llm_amd.engine.llm import LLM, CacheConfig
    from tinyserve_llm_amd.engine.scheduler import SchedulerConfig
    from tinyserve_llm_amd.engine.sequence import SamplingParams
    base = dict(max_model_len=128, max_num_seqs=8, max_num_batched_tokens=80, max_prefill_chunk=32, watermark=0.0)
    prompts = [prompt(70 + i, 3 + 5 * i, 384) for i in range(11)]
    params = [SamplingParams(max_tokens=3 + 4 * (i % 6), temperature=1.5 if i % 3 else 0.0, n=2 if i == 4 else 1,
                             ignore_eos=i % 2 == 0) for i in range(11)]
    # an end token that some request draws in the middle of its output: found with a token nobody draws
    free = LLM(folder_b, SchedulerConfig(eos_token_id=10 ** 6, **base), CacheConfig(block_size=16), dtype=torch.float32,
               num_blocks=120, seed=11, run_ahead=False)
    drawn = [r.token_ids[0] for r, p in zip(free.generate(prompts, params), params) if not p.ignore_eos]
    eos = next(out[len(out) // 2] for out in drawn if len(out) >= 5)
    sc = SchedulerConfig(eos_token_id=eos, **base)
    outs, stats = [], []
    for ahead in (True, False):
        llm = LLM(folder_b, sc, CacheConfig(block_size=16), dtype=torch.float32, num_blocks=num_blocks, seed=11,
                  run_ahead=ahead)
        outs.append([(r.token_ids, r.finish_reasons) for r in llm.generate(prompts, params)])
        stats.append(llm.scheduler.stats())
        assert llm.manager.stats().blocks_in_use == 0 and llm._ahead is None
    assert outs[0] == outs[1]
    assert any("eos" in reasons for _, reasons in outs[0]) and any("length" in reasons for _, reasons in outs[0])
    if num_blocks == 18:
        assert stats[0].preemptions > 0 and stats[1].preemptions > 0


def test_streaming_copies_of_the_weights_change_nothing(tmp_path):
    """Layers may keep their weights once more in the decode kernels' reading order; decode steps
    read the copies, steps with many rows the weights themselves. Same tokens either way. (A width of
    256 is the least the weight-streaming kernel takes; the tiny configurations never reach it.)"""
    from tinyserve_llm_amd.config import LlamaConfig
    from tinyserve_llm_amd.engine.llm import LLM, CacheConfig
    from tinyserve_llm_amd.engine.scheduler import SchedulerConfig
    from tinyserve_llm_amd.engine.sequence import SamplingParams
    from tinyserve_llm_amd.weights.random_init import write_random_model
    config = LlamaConfig(vocab_size=300, hidden_size=256, intermediate_size=512, num_hidden_layers=2,
                         num_attention_heads=4, num_key_value_heads=2, head_dim=64, max_position_embeddings=256,
                         rms_norm_eps=1e-5, rope_theta=10000.0, rope_scaling=None, tie_word_embeddings=True, eos_token_id=299)
    write_random_model(str(tmp_path), config, 4, torch.bfloat16)
    sc = SchedulerConfig(max_model_len=128, max_num_seqs=8, max_num_batched_tokens=80)
    prompts = [prompt(90 + i, 4 + 9 * i, 300) for i in range(5)]
    outs = []
    for keep in (True, False):
        llm = LLM(str(tmp_path), sc, CacheConfig(block_size=16), dtype=torch.bfloat16, num_blocks=60, seed=2,
                  keep_streaming_copies=keep)
        mixer, ff = llm.model.layers[0].mixer, llm.model.layers[0].feed_forward
        assert (mixer.qkv_rope_packed is not None) == keep and (mixer.o_packed is not None) == keep
        assert (ff.gate_up_packed is not None) == keep and (ff.down_packed is not None) == keep
        outs.append([r.token_ids for r in llm.generate(prompts, SamplingParams(max_tokens=10, temperature=0.7, ignore_eos=True))])
    assert outs[0] == outs[1]
    plain = PlainLlama(str(tmp_path), torch.float64)
    got = LLM(str(tmp_path), sc, CacheConfig(block_size=16), dtype=torch.float32, num_blocks=60).generate(
        prompts[:2], SamplingParams(max_tokens=6, temperature=0.0, ignore_eos=True))
    assert [r.token_ids[0] for r in got] == [plain.greedy(p, 6) for p in prompts[:2]]


def test_recorded_steps_with_library_products_replay_what_eager_steps_compute(tmp_path):
    """Above 32 requests a decode step's projections go to the vendor's matrix library, inside the
    recorded graph as well. In bfloat16 the graph's replays (several, with prompts run eagerly in
    between, and again in a second round of requests) must give the tokens of the engine that runs
    every step eagerly: the same kernels on the same numbers."""
    from tinyserve_llm_amd.config import LlamaConfig
    from tinyserve_llm_amd.engine.llm import LLM, CacheConfig
    from tinyserve_llm_amd.engine.scheduler import SchedulerConfig
    from tinyserve_llm_amd.engine.sequence import SamplingParams
    from tinyserve_llm_amd.weights.random_init import write_random_model
    config = LlamaConfig(vocab_size=300, hidden_size=256, intermediate_size=512, num_hidden_layers=2,
                         num_attention_heads=4, num_key_value_heads=2, head_dim=64, max_position_embeddings=256,
                         rms_norm_eps=1e-5, rope_theta=10000.0, rope_scaling=None, tie_word_embeddings=True, eos_token_id=299)
    write_random_model(str(tmp_path), config, 6, torch.bfloat16)
    sc = SchedulerConfig(max_model_len=96, max_num_seqs=48, max_num_batched_tokens=256)
    prompts = [prompt(300 + i, 3 + i % 11, 300) for i in range(44)]
    params = [SamplingParams(max_tokens=5 + i % 7, temperature=0.0, ignore_eos=True) for i in range(44)]
    outs = []
    for graphs in (True, False):
        llm = LLM(str(tmp_path), sc, CacheConfig(block_size=16), dtype=torch.bfloat16, num_blocks=300, seed=1,
                  decode_graphs=graphs)
        outs.append([r.token_ids for r in llm.generate(prompts, params)])
        if graphs:
            sizes = sorted({size for size, width in llm.runner.graphs.graphs})
            assert max(sizes) > 32, f"a batch above 32 requests was recorded: {sizes}"
            assert [r.token_ids for r in llm.generate(prompts, params)] == outs[0]
    assert outs[0] == outs[1]


@pytest.mark.parametrize("hidden,inter,vocab,heads,kv,hd", [(100, 150, 333, 5, 5, 16), (104, 152, 1001, 6, 2, 48),
                                                             (36, 20, 77, 3, 1, 16)])
def test_awkward_sizes_run_in_both_precisions(tmp_path, hidden, inter, vocab, heads, kv, hd):
    """Widths whose rows are not 16-byte aligned, odd vocabularies, head counts that divide nothing:
    the kernels' general forms serve them (or the vector forms, where a size happens to allow),
    never a wrong result. A prompt in two portions against the plain model, float32 and bfloat16."""
    from tinyserve_llm_amd.config import LlamaConfig
    from tinyserve_llm_amd.engine.llm import LLM, CacheConfig
    from tinyserve_llm_amd.engine.runner import StepEntry
    from tinyserve_llm_amd.engine.scheduler import SchedulerConfig
    from tinyserve_llm_amd.weights.random_init import write_random_model
    config = LlamaConfig(vocab_size=vocab, hidden_size=hidden, intermediate_size=inter, num_hidden_layers=2,
                         num_attention_heads=heads, num_key_value_heads=kv, head_dim=hd, max_position_embeddings=128,
                         rms_norm_eps=1e-5, rope_theta=10000.0, rope_scaling=None, tie_word_embeddings=True,
                         eos_token_id=vocab - 1)
    write_random_model(str(tmp_path), config, 3, torch.float32)
    ids = prompt(7, 70, vocab)
    sc = SchedulerConfig(max_model_len=128, max_num_seqs=4, max_num_batched_tokens=256)
    for dtype, tolerance in ((torch.float32, 2e-5), (torch.bfloat16, 3e-2)):
        want = PlainLlama(str(tmp_path), torch.float64, weights_as=None if dtype == torch.float32 else dtype).logits(ids)
        llm = LLM(str(tmp_path), sc, CacheConfig(block_size=16), dtype=dtype, num_blocks=20)
        llm.manager.allocate(0, ids[:40])
        first = llm.runner.step([StepEntry(0, ids[:40], 0, list(range(40)))])
        llm.manager.commit(0, 40)
        llm.manager.append_slots(0, ids[40:])
        rest = llm.runner.step([StepEntry(0, ids[40:], 40, list(range(30)))])
        got = torch.cat([first, rest]).double().cpu()
        spread = float(want.max() - want.min())
        assert float((got - want).abs().max()) <= tolerance * spread, f"{dtype}: {float((got - want).abs().max())} of {spread}"


def test_small_portions_over_a_long_context_walk_the_keys_in_chunks(tmp_path):
    """Behind 2,500 cached tokens the next portions are small: too few tiles to fill the chip, so
    the bfloat16 attention kernel cuts each tile's keys into chunks and combines them. A portion of
    60 alone, then one of 40 behind another request's decoded token (which goes to the decode
    kernel in the same step), against the plain model over the whole prompt."""
    from tinyserve_llm_amd.config import LlamaConfig
    from tinyserve_llm_amd.engine.llm import LLM, CacheConfig
    from tinyserve_llm_amd.engine.runner import StepEntry
    from tinyserve_llm_amd.engine.scheduler import SchedulerConfig
    from tinyserve_llm_amd.ops import hip
    from tinyserve_llm_amd.weights.random_init import write_random_model
    config = LlamaConfig(vocab_size=300, hidden_size=128, intermediate_size=192, num_hidden_layers=2,
                         num_attention_heads=4, num_key_value_heads=2, head_dim=64, max_position_embeddings=4096,
                         rms_norm_eps=1e-5, rope_theta=10000.0, rope_scaling=None, tie_word_embeddings=True,
                         eos_token_id=299)
    write_random_model(str(tmp_path), config, 5, torch.float32)
    ids, other = prompt(11, 2600, 300), prompt(12, 31, 300)
    assert hip.prefill_splits(2 * 2, 2560)[0] > 1, "the step below is one the plan cuts"
    sc = SchedulerConfig(max_model_len=4096, max_num_seqs=4, max_num_batched_tokens=4096)
    for dtype, tolerance in ((torch.float32, 2e-5), (torch.bfloat16, 3e-2)):
        plain = PlainLlama(str(tmp_path), torch.float64, weights_as=None if dtype == torch.float32 else dtype)
        want, want_other = plain.logits(ids), plain.logits(other)
        llm = LLM(str(tmp_path), sc, CacheConfig(block_size=64), dtype=dtype, num_blocks=48)
        llm.manager.allocate(0, ids[:2500])
        llm.manager.allocate(1, other[:30])
        llm.runner.step([StepEntry(0, ids[:2500], 0, []), StepEntry(1, other[:30], 0, [])])
        llm.manager.commit(0, 2500)
        llm.manager.commit(1, 30)
        llm.manager.append_slots(0, ids[2500:2560])
        alone = llm.runner.step([StepEntry(0, ids[2500:2560], 2500, list(range(60)))])
        llm.manager.commit(0, 60)
        llm.manager.append_slots(0, ids[2560:])
        llm.manager.append_slots(1, other[30:])
        mixed = llm.runner.step([StepEntry(1, other[30:], 30, [0]), StepEntry(0, ids[2560:], 2560, list(range(40)))])
        got = torch.cat([alone, mixed[1:]]).double().cpu()
        spread = float(want.max() - want.min())
        assert float((got - want[2500:]).abs().max()) <= tolerance * spread, f"{dtype}: {float((got - want[2500:]).abs().max())} of {spread}"
        assert float((mixed[0].double().cpu() - want_other[30]).abs().max()) <= tolerance * spread


def test_the_engines_own_tiled_products_serve_steps_of_many_rows(tmp_path):
    """With `many_rows_products("tiled")` a prompt's projections, its gated feed-forward and its
    head run on the engine's own tiled kernel instead of the vendor library: the logits of a prompt
    in two portions against the plain model, and the same tokens generated as with the library."""
    from tinyserve_llm_amd.config import LlamaConfig
    from tinyserve_llm_amd.engine.llm import LLM, CacheConfig
    from tinyserve_llm_amd.engine.runner import StepEntry
    from tinyserve_llm_amd.engine.scheduler import SchedulerConfig
    from tinyserve_llm_amd.ops import hip
    from tinyserve_llm_amd.weights.random_init import write_random_model
    config = LlamaConfig(vocab_size=300, hidden_size=128, intermediate_size=192, num_hidden_layers=2,
                         num_attention_heads=4, num_key_value_heads=2, head_dim=32, max_position_embeddings=256,
                         rms_norm_eps=1e-5, rope_theta=10000.0, rope_scaling=None, tie_word_embeddings=False,
                         eos_token_id=299)
    write_random_model(str(tmp_path), config, 9, torch.bfloat16)
    ids = prompt(21, 150, 300)
    want = PlainLlama(str(tmp_path), torch.float64, weights_as=torch.bfloat16).logits(ids)
    sc = SchedulerConfig(max_model_len=256, max_num_seqs=4, max_num_batched_tokens=256)
    calls = []
    tiled = hip.gemm_tiled
    try:
        hip.many_rows_products("tiled")
        hip.gemm_tiled = lambda *a, **k: (calls.append(k.get("glu", False)), tiled(*a, **k))[1]
        llm = LLM(str(tmp_path), sc, CacheConfig(block_size=16), dtype=torch.bfloat16, num_blocks=20)
        llm.manager.allocate(0, ids[:90])
        first = llm.runner.step([StepEntry(0, ids[:90], 0, list(range(90)))])
        llm.manager.commit(0, 90)
        llm.manager.append_slots(0, ids[90:])
        rest = llm.runner.step([StepEntry(0, ids[90:], 90, list(range(60)))])
        llm.manager.commit(0, 60)
        llm.manager.release(0)
        assert calls.count(True) == 4 and calls.count(False) == 2 * (2 * 3 + 1), "gate_up twice per layer; qkv, o, down and the head"
        got = torch.cat([first, rest]).double().cpu()
        spread = float(want.max() - want.min())
        assert float((got - want).abs().max()) <= 3e-2 * spread
        own = [c.token_ids for c in llm.generate([ids[:50], ids[50:120]], greedy(8))]
    finally:
        hip.gemm_tiled = tiled
        hip.many_rows_products("library")
    llm = LLM(str(tmp_path), sc, CacheConfig(block_size=16), dtype=torch.bfloat16, num_blocks=20)
    lib = [c.token_ids for c in llm.generate([ids[:50], ids[50:120]], greedy(8))]
    plain = PlainLlama(str(tmp_path), torch.float64, weights_as=torch.bfloat16)
    for p_, a_, b_ in zip((ids[:50], ids[50:120]), own, lib):
        if a_ != b_:      # a draw between two close logits may fall either way in bfloat16: then both must be close calls
            at = next(i for i, (x_, y_) in enumerate(zip(a_, b_)) if x_ != y_)
            row = plain.logits(p_ + a_[:at])[-1]
            assert float(row.max() - row[[a_[at], b_[at]]].min()) <= 3e-2 * float(row.max() - row.min())


@pytest.mark.parametrize("case", range(10))
def test_random_workloads_generate_the_same_under_every_engine_setting(case, folder_a, folder_b):
    """Random requests (shared prefixes, forks, sampling, end tokens, lengths), page sizes, pools
    so small that sequences are preempted, token budgets, portions: recorded or eager decode steps,
    steps closed in two halves or in one, prefix cache on or off must all generate the same tokens
    in float32."""
    import random

    from tinyserve_llm_amd.engine.llm import LLM, CacheConfig
    from tinyserve_llm_amd.engine.scheduler import SchedulerConfig
    from tinyserve_llm_amd.engine.sequence import SamplingParams
    rng = random.Random(1000 + case)
    folder, vocab = (folder_a, 256) if rng.random() < 0.5 else (folder_b, 384)
    shared = prompt(2000 + case, rng.randint(0, 40), vocab - 1)
    prompts, params = [], []
    for i in range(rng.randint(3, 24)):
        prompts.append((shared if rng.random() < 0.4 else []) + prompt(case * 100 + i, rng.randint(1, 60), vocab - 1))
        params.append(SamplingParams(max_tokens=rng.randint(1, 20), temperature=rng.choice([0.0, 0.0, 0.8]),
                                     n=rng.choice([1, 1, 1, 2, 3]), ignore_eos=rng.random() < 0.5))
    page = rng.choice([4, 8, 16])
    need = max(-(-(len(p) + sp.max_tokens) // page) * sp.n for p, sp in zip(prompts, params))
    blocks = rng.choice([need + 2, need * 2, need * 6, 400])
    seqs = rng.choice([4, 8, 40])
    sc = SchedulerConfig(max_model_len=128, max_num_seqs=seqs, max_num_batched_tokens=max(rng.choice([64, 128, 512]), seqs + 1),
                         max_prefill_chunk=rng.choice([0, 0, 7, 32]), watermark=0.0)
    outs = []
    for graphs, ahead, caching in ((False, False, False), (True, True, True), (True, False, False), (False, True, True)):
        llm = LLM(folder, sc, CacheConfig(block_size=page, caching=caching), dtype=torch.float32, num_blocks=blocks, seed=case,
                  decode_graphs=graphs, run_ahead=ahead)
        outs.append([(c.token_ids, c.finish_reasons) for c in llm.generate(prompts, params)])
        assert caching or llm.manager.num_available_blocks() == llm.manager.num_blocks, "pages leaked"
    assert outs[1] == outs[0] and outs[2] == outs[0] and outs[3] == outs[0]


def test_recorded_steps_are_bounded_and_dropping_them_changes_nothing(folder_b):
    """At most `max_decode_graphs` recorded steps are kept, the one replayed longest ago goes first,
    and their own buffers stay inside the budget; walking many (batch size, context) keys twice
    leaves the device's memory where the first walk left it, and an engine that keeps only three
    graphs generates what an engine without graphs does."""
    from tinyserve_llm_amd.engine.llm import LLM, CacheConfig
    from tinyserve_llm_amd.engine.scheduler import SchedulerConfig
    from tinyserve_llm_amd.engine.sequence import SamplingParams
    sc = SchedulerConfig(max_model_len=320, max_num_seqs=40, max_num_batched_tokens=160, max_prefill_chunk=32)
    llm = LLM(folder_b, sc, CacheConfig(block_size=16), dtype=torch.float32, num_blocks=400, seed=5, max_decode_graphs=6,
              record_decode_steps=[3, (9, 100)])
    graphs = llm.runner.graphs
    assert list(graphs.graphs) == [(3, 32), (16, 16)], "recorded at start: 320 positions reach 512 in pages of 16; 9 requests in 16 rows"
    keys = [(batch, context) for context in (60, 300) for batch in (1, 2, 3, 4, 5, 6, 7, 8, 9, 17, 25, 33)]
    held = []
    for walk in range(2):
        for batch, context in keys:
            key = graphs.record(batch, context)
            assert key in graphs.graphs and len(graphs.graphs) <= 6 and list(graphs.graphs)[-1] == key
            assert graphs.memory_held() <= graphs.memory_budget
        torch.cuda.synchronize()
        held.append(torch.cuda.memory_allocated())
    assert graphs.recorded >= 2 * len(keys) - 6 and graphs.dropped == graphs.recorded - 6, (graphs.recorded, graphs.dropped)
    assert held[1] <= held[0], f"the second walk took more memory: {held}"
    # a budget of bytes: graphs of 40 rows hold 40 x 384 logits each; room for two of them
    tight = LLM(folder_b, sc, CacheConfig(block_size=16), dtype=torch.float32, num_blocks=400, seed=5,
                decode_graph_memory=2 * 40 * 384 * 4 + 4096)
    for context in (10, 300, 10, 300):
        tight.runner.graphs.record(40, context)
        tight.runner.graphs.record(33, context)       # the same graph: 40 rows
        tight.runner.graphs.record(1, context)
    assert tight.runner.graphs.memory_held() <= tight.runner.graphs.memory_budget and tight.runner.graphs.dropped > 0
    prompts = [prompt(70 + i, 3 + 5 * i, 384) for i in range(11)]
    params = [SamplingParams(max_tokens=3 + 2 * (i % 6), temperature=0.7 if i % 3 == 0 else 0.0, ignore_eos=True) for i in range(11)]
    outs = []
    for cap in (3, None):
        one = LLM(folder_b, sc, CacheConfig(block_size=16), dtype=torch.float32, num_blocks=400, seed=5,
                  decode_graphs=cap is not None, max_decode_graphs=cap or 64)
        outs.append([r.token_ids for r in one.generate(prompts, params)])
        if cap:
            assert one.runner.graphs.dropped > 0 and len(one.runner.graphs.graphs) <= cap
    assert outs[0] == outs[1]


def test_drawn_tokens_say_when_the_graph_has_overwritten_them(folder_a):
    """The tokens of a replayed step stay on the device until the graph's next replay and in one of
    two landing places on the host until the replay after that; a result held longer refuses to be
    read instead of handing out another step's tokens."""
    from tinyserve_llm_amd.engine.runner import DrawnTokens, StepEntry, StepError
    llm = engine(folder_a)
    m, r = llm.manager, llm.runner
    ids = prompt(3, 9, 256)
    m.allocate(0, ids)
    r.step([StepEntry(0, ids, 0, [])])
    m.commit(0, len(ids))
    held = []
    for k in range(3):
        m.append_slots(0, [5 + k])
        held.append(r.step_sample([StepEntry(0, [5 + k], len(ids) + k, [0])], [0.0], [k], llm.seed))
        m.commit(0, 1)
    assert all(isinstance(h, DrawnTokens) for h in held)
    assert len(held[2].tolist()) == 1 and len(held[1].tolist()) == 1 and held[2].on_device.shape == (1,)
    with pytest.raises(StepError, match="replayed twice"):
        held[0].tolist()
    with pytest.raises(StepError, match="replayed since"):
        held[1].on_device
    m.release(0)


def test_without_library_timing_two_processes_draw_the_same_bfloat16_tokens(tmp_path):
    """Steps of more than 64 requests take their projections from the vendor's matrix library. With
    its candidates timed, which of them serves a shape may differ from run to run; with the timing
    off (`--no-library-timing`) every shape keeps the library's first candidate, the record says
    so, and two processes generate the same tokens."""
    from tinyserve_llm_amd.config import LlamaConfig
    from tinyserve_llm_amd.weights.random_init import write_random_model
    config = LlamaConfig(vocab_size=300, hidden_size=256, intermediate_size=512, num_hidden_layers=2,
                         num_attention_heads=4, num_key_value_heads=2, head_dim=64, max_position_embeddings=256,
                         rms_norm_eps=1e-5, rope_theta=10000.0, rope_scaling=None, tie_word_embeddings=True, eos_token_id=299)
    folder = write_random_model(str(tmp_path / "m"), config, 6, torch.bfloat16)
    records = []
    for run in range(2):
        out = str(tmp_path / f"r{run}.json")
        cmd = [sys.executable, "-m", "tinyserve_llm_amd.generate", "--model", folder, "--prompt-lengths",
               ",".join(str(3 + i % 11) for i in range(80)), "--max-tokens", "6", "--temperature", "0.8", "--ignore-eos",
               "--block-size", "16", "--num-blocks", "400", "--max-model-len", "96", "--max-num-seqs", "96",
               "--max-num-batched-tokens", "512", "--no-library-timing", "--out", out]
        r = subprocess.run(cmd, cwd=ROOT, capture_output=True, text=True, timeout=300)
        assert r.returncode == 0, r.stderr[-2000:]
        with open(out) as f:
            records.append(json.load(f))
    a, b = records
    assert a["library_choices"] and all(c["chosen"] == "first" for c in a["library_choices"]), a["library_choices"]
    assert any(c["rows"] > 64 for c in a["library_choices"]), "a step of many requests went through the library"
    assert a["library_choices"] == b["library_choices"]
    assert [c["token_ids"] for c in a["completions"]] == [c["token_ids"] for c in b["completions"]]

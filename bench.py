"""Decode and prefill throughput of the Llama-3.2-1B shape with random weights on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A "step" is one decode step of the whole engine (scheduler, step function, kernels, sampling) at
batch 8 with 2,048-token contexts that grow while decoding. Prints ONE JSON line. The same line
carries the 2,048-token prefill, the decode step's HBM roofline, and decode at batch 1 and 64.

    python bench.py --kernel-classes [--batch B]

times the kernels of one decode step class by class (qkv, attention, o, gate|up, down, norms, head,
sampling) with events around each launch of an eager step, and prints the bytes each class has to
read, its time and its rate beside the step's total, as one JSON line.

    python bench.py --scenario requests-3b | chunked-8b [--layers L]

runs a whole workload through `LLM.generate` instead and prints one JSON line of its own: many
requests that arrive together, at the layer sizes of Llama 3.2 3B (prompts of 512 to 4,096 tokens, a
quarter of them behind a common 1,024-token prefix, prefix cache on) or of Llama 3.1 8B (8,192-token
contexts whose prompts are fed in portions of 2,048 tokens beside the decoding requests).
"""

from __future__ import annotations

import argparse
import json
import os
import random
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# MI355X published peaks
HBM_BYTES_PER_S = 8.0e12
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}

# layer sizes (--shape); the default, "1b", is the one the headline numbers are quoted on
SHAPES = {
    "1b": dict(model="llama-3.2-1b-shape", layers_full=16, rope_factor=32.0,
               shape=dict(vocab_size=128256, hidden_size=2048, intermediate_size=8192, num_attention_heads=32,
                          num_key_value_heads=8, head_dim=64, max_position_embeddings=131072, rms_norm_eps=1e-5,
                          rope_theta=500000.0, tie_word_embeddings=True)),
    "3b": dict(model="llama-3.2-3b-shape", layers_full=28, rope_factor=32.0,
               shape=dict(vocab_size=128256, hidden_size=3072, intermediate_size=8192, num_attention_heads=24,
                          num_key_value_heads=8, head_dim=128, max_position_embeddings=131072, rms_norm_eps=1e-5,
                          rope_theta=500000.0, tie_word_embeddings=True)),
    "8b": dict(model="llama-3.1-8b-shape", layers_full=32, rope_factor=8.0,
               shape=dict(vocab_size=128256, hidden_size=4096, intermediate_size=14336, num_attention_heads=32,
                          num_key_value_heads=8, head_dim=128, max_position_embeddings=131072, rms_norm_eps=1e-5,
                          rope_theta=500000.0, tie_word_embeddings=False)),
}
ROPE = dict(factor=32.0, low_freq_factor=1.0, high_freq_factor=4.0, original_max_position_embeddings=8192)
PROMPT_LEN, MAX_MODEL_LEN, PAGE = 2048, 4096, 256
SHAPE = SHAPES["1b"]["shape"]

# whole workloads: layer sizes, requests, and how the scheduler is set for them
SCENARIOS = {
    "requests-3b": dict(**SHAPES["3b"], requests=64, prompt=(512, 4096), shared=(0.25, 1024), decode=256, budget=8192,
                        chunk=0, caching=True),
    "chunked-8b": dict(**SHAPES["8b"], requests=32, prompt=(7936, 7936), shared=(0.0, 0), decode=256,
                       budget=2048 + 32, chunk=2048, caching=False),
}


def scenario(name: str, layers: int | None, dtype_name: str) -> int:
    """One workload from first request to last token through `LLM.generate`; one JSON line."""
    import torch

    from tinyserve_llm_amd.config import LlamaConfig, RopeScaling
    from tinyserve_llm_amd.engine.llm import LLM, CacheConfig
    from tinyserve_llm_amd.engine.loading import random_model
    from tinyserve_llm_amd.engine.scheduler import SchedulerConfig
    from tinyserve_llm_amd.engine.sequence import SamplingParams

    w = SCENARIOS[name]
    layers = layers or w["layers_full"]
    config = LlamaConfig(num_hidden_layers=layers, rope_scaling=RopeScaling(**{**ROPE, "factor": w["rope_factor"]}),
                         **w["shape"])
    dtype = torch.bfloat16 if dtype_name == "bf16" else torch.float32
    model = random_model(config, 0, dtype, "cuda:0")
    rng = random.Random(0)
    lo, hi = w["prompt"]
    share, prefix_len = w["shared"]
    prefix = [rng.randrange(config.vocab_size) for _ in range(prefix_len)]
    prompts = []
    for i in range(w["requests"]):
        n = rng.randint(lo, hi)
        head = prefix if i < share * w["requests"] and n > prefix_len else []
        prompts.append(head + [rng.randrange(config.vocab_size) for _ in range(n - len(head))])
    rng.shuffle(prompts)
    max_len = hi + w["decode"]
    pages = sum(-(-(len(p) + w["decode"]) // PAGE) for p in prompts) + 8
    sc = SchedulerConfig(max_model_len=max_len, max_num_seqs=w["requests"], max_num_batched_tokens=w["budget"],
                         max_prefill_chunk=w["chunk"])
    sp = SamplingParams(max_tokens=w["decode"], temperature=0.0, ignore_eos=True)

    def run(subset) -> tuple[float, LLM]:
        llm = LLM(None, sc, CacheConfig(block_size=PAGE, caching=w["caching"]), dtype=dtype, num_blocks=pages,
                  seed=0, model=model)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        llm.generate(subset, sp)
        torch.cuda.synchronize()
        return time.perf_counter() - t0, llm

    # once untimed, with other tokens of the same lengths: libraries pick and time their kernels for
    # the batch sizes the workload meets (kept for the process); the timed run has a fresh engine
    cold_seconds, cold = run([[rng.randrange(config.vocab_size) for _ in p] for p in prompts])
    recorded_cold = cold.runner.graphs.recorded if cold.runner.graphs is not None else 0
    del cold
    seconds, llm = run(prompts)
    st, cs = llm.scheduler.stats(), llm.manager.stats()
    portions = [r for r in llm.steps if r.num_tokens > r.num_seqs]
    decodes = [r for r in llm.steps if r.num_tokens == r.num_seqs]
    prompt_tokens = sum(len(p) for p in prompts)
    record = {
        "metric": f"tokens/s of a whole workload ({name})", "value": (prompt_tokens + st.decode_tokens) / seconds,
        "unit": "tokens/s", "n_gpus": 1, "seconds": seconds, "steps": len(llm.steps), "higher_is_better": True,
        # the same workload's first run in the process: decode steps recorded as their batch sizes are first met,
        # the matrix library's candidates timed once per shape
        "cold_seconds": cold_seconds, "decode_steps_recorded_cold": recorded_cold,
        "dtype": dtype_name, "data": "synthetic uniform token ids, random weights N(0,0.02)",
        "output_tokens_per_s": st.decode_tokens / seconds, "prompt_tokens": prompt_tokens,
        "prefilled_tokens": st.prefill_tokens, "cached_tokens": st.cached_tokens, "output_tokens": st.decode_tokens,
        "preemptions": st.preemptions, "evictions": cs.evictions,
        "steps_with_prompt_portions": {"steps": len(portions), "seconds": sum(r.end - r.start for r in portions),
                                       "tokens": sum(r.num_tokens for r in portions)},
        "steps_of_decodes_only": {"steps": len(decodes), "seconds": sum(r.end - r.start for r in decodes),
                                  "tokens": sum(r.num_tokens for r in decodes)},
        "config": {"model": w["model"], "layers": layers, "layers_full": w["layers_full"],
                   "hidden": config.hidden_size, "heads": config.num_attention_heads,
                   "kv_heads": config.num_key_value_heads, "head_dim": config.head_dim,
                   "intermediate": config.intermediate_size, "vocab": config.vocab_size, "requests": w["requests"],
                   "prompt_min": lo, "prompt_max": hi, "shared_prefix": prefix_len, "decode_tokens": w["decode"],
                   "token_budget": w["budget"], "prefill_chunk": w["chunk"], "page_size": PAGE, "pages": pages},
    }
    print(json.dumps(record))
    return 0


def kernel_classes(llm, config, batch: int, reps: int = 5) -> dict:
    """Times one decode step's kernels by class. An eager step (no graph) is run once with every
    launch of the engine's kernel module noted down with its operands; then each class's launches
    (one per layer, with that layer's own weights) are recorded into a graph of their own, and the
    graph is replayed between two events after a sweep of the caches: a class's time is its kernels
    and the dispatches between them, as a recorded decode step sees them. Its bytes are what it has
    to read once (weights, or the keys and values of the live requests). The best of `reps` replays."""
    import torch

    from tinyserve_llm_amd.ops import hip

    c = config
    item = 2 if llm.dtype == torch.bfloat16 else 4
    by_shape = {(c.q_size + 2 * c.kv_size, c.hidden_size): "qkv", (c.hidden_size, c.q_size): "o",
                (2 * c.intermediate_size, c.hidden_size): "gate_up", (c.hidden_size, c.intermediate_size): "down",
                (c.vocab_size, c.hidden_size): "head"}
    calls: dict[str, list] = {}

    def note(klass, nbytes, inner, a, kw):
        calls.setdefault(klass, []).append((nbytes, inner, a, kw))
        return inner(*a, **kw)

    def product(name, weight_of):
        inner = getattr(hip, name)

        def noted(*a, **kw):
            w = weight_of(*a, **kw)
            if w.dim() == 4:                                   # a streaming copy: [N / 16, K / 32, 64, 8]
                shape = (w.shape[0] * 16, w.shape[1] * 32)
            elif w.dim() == 5:                                 # the 8-row form's: [N / 8, waves, steps, 64, 8]
                shape = (w.shape[0] * 8, w.shape[1] * w.shape[2] * 64)
            else:
                shape = tuple(w.shape)
            # (a copy's rows are padded to whole tiles)
            klass = next((v for k, v in by_shape.items() if k[1] == shape[1] and 0 <= shape[0] - k[0] < 16), f"product {shape}")
            return note(klass, shape[0] * shape[1] * item, inner, a, kw)
        return noted

    def other(name, klass, nbytes_of=lambda *a, **kw: 0):
        inner = getattr(hip, name)
        return lambda *a, **kw: note(klass, nbytes_of(*a, **kw), inner, a, kw)

    live = sum(s.num_tokens for s in llm.scheduler.running)
    kv_layer = live * 2 * c.kv_size * item
    patched = {
        "gemm_skinny": product("gemm_skinny", lambda x, w, *a, **kw: w),
        "gemm_skinny8": product("gemm_skinny8", lambda x, w, *a, **kw: w),
        "gemm_rows64": product("gemm_rows64", lambda x, packed, *a, **kw: packed),
        "gemm_rows64_sliced": product("gemm_rows64_sliced", lambda x, packed, *a, **kw: packed),
        "qkv_rope_store_sliced": product("qkv_rope_store_sliced", lambda x, packed, *a, **kw: packed),
        "gemm_library": product("gemm_library", lambda x, w, *a, **kw: w),
        "gemm_exact": product("gemm_exact", lambda x, w, *a, **kw: w),
        "qkv_rope_store": product("qkv_rope_store", lambda x, w, *a, **kw: w),
        "paged_attention_decode": other("paged_attention_decode", "attention", lambda *a, **kw: kv_layer),
        "paged_attention_wave": other("paged_attention_wave", "attention", lambda *a, **kw: kv_layer),
        "rmsnorm": other("rmsnorm", "norm"), "rope_store": other("rope_store", "rotation and cache write"),
        "silu_mul": other("silu_mul", "gate"), "sample": other("sample", "sampling"), "embedding": other("embedding", "embedding"),
    }
    kept = {name: getattr(hip, name) for name in patched}
    graphs, llm.runner.graphs, ahead = llm.runner.graphs, None, llm.run_ahead
    llm.run_ahead = False
    try:
        llm.step()                                         # (closes the step that was started ahead, starts none)
        for name, fn in patched.items():
            setattr(hip, name, fn)
        llm.step()
        torch.cuda.synchronize()
    finally:
        for name, fn in kept.items():
            setattr(hip, name, fn)
        llm.runner.graphs, llm.run_ahead = graphs, ahead
    sweep = torch.zeros(128 << 20, dtype=torch.int32, device="cuda")       # 512 MB: more than the caches hold
    begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    classes: dict[str, dict] = {}
    tiny = torch.zeros(64, dtype=torch.int32, device="cuda")
    calls = {"(a graph of one small kernel)": [(0, lambda: tiny.add_(1), (), {})], **calls}
    overhead = 0.0
    with torch.inference_mode():                          # (the step's tensors were made under it)
        for klass, noted in calls.items():
            for _, inner, a, kw in noted:                      # once outside a recording (libraries set themselves up)
                inner(*a, **kw)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                outs = [inner(*a, **kw) for _, inner, a, kw in noted]
            times = []
            for _ in range(reps + 1):
                sweep.sum()                                    # read, not written: the caches hold nothing of the weights, and nothing dirty
                begin.record()
                graph.replay()
                end.record()
                end.synchronize()
                times.append(1e3 * begin.elapsed_time(end))
            del outs, graph
            us, nbytes = max(min(times[1:]) - overhead, 1e-3), sum(n for n, *_ in noted)     # (a class of one tiny kernel may cost no more than the replay itself)
            if klass.startswith("("):
                overhead = us                                  # what a replay costs before its first kernel's work: taken off every class
                continue
            classes[klass] = {"launches": len(noted), "bytes": nbytes, "us": us, "us_per_launch": us / len(noted),
                              "GBps": nbytes / us / 1e3, "frac_of_hbm": nbytes / us * 1e6 / HBM_BYTES_PER_S}
    total = {"bytes": sum(r["bytes"] for r in classes.values()), "us": sum(r["us"] for r in classes.values())}
    total["GBps"] = total["bytes"] / total["us"] / 1e3
    return {"batch": batch, "live_tokens": live, "classes": dict(sorted(classes.items(), key=lambda kv: -kv[1]["us"])),
            "all_classes": total, "replay_overhead_us": overhead}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=None)
    ap.add_argument("--shape", default="1b", choices=sorted(SHAPES), help="layer sizes of the decode and prefill steps")
    ap.add_argument("--context", type=int, default=PROMPT_LEN,
                    help="tokens of every prompt: the decode steps start from contexts of this length, and the prefill "
                         "is of this many tokens (the headline numbers are quoted at the default)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--points", default="1,64", help="further decode batch sizes (comma-separated; '' for none)")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--only", default="all", choices=["all", "prefill"],
                    help="'prefill': time the 2,048-token prefill alone and print its record (for profiling)")
    ap.add_argument("--scenario", default=None, choices=sorted(SCENARIOS),
                    help="run a whole workload through LLM.generate instead of the decode step")
    ap.add_argument("--kernel-classes", action="store_true",
                    help="time one decode step's kernels class by class (bytes, microseconds, GB/s) and exit")
    ap.add_argument("--peaks", action="store_true",
                    help="measure what a kernel that only reads memory and a loop of matrix instructions reach on "
                         "this GPU, print them beside the published peaks and exit")
    ap.add_argument("--many-rows-products", default="library", choices=["library", "tiled"],
                    help="bfloat16 products of many rows: the vendor's library, or the engine's own tiled kernel")
    args = ap.parse_args()
    if args.many_rows_products != "library":
        from tinyserve_llm_amd.ops import hip
        hip.many_rows_products(args.many_rows_products)
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported by this engine")
        return 2
    if args.peaks:
        from tinyserve_llm_amd.ops import hip
        measured = hip.measure_peaks()
        print(json.dumps({"peaks": {"read": {"measured": measured["read_GBps"], "published": HBM_BYTES_PER_S / 1e9, "unit": "GB/s"},
                                    "mfma_bf16": {"measured": measured["mfma_bf16_TFLOPs"], "published": PEAK_FLOPS["bf16"] / 1e12,
                                                  "unit": "TFLOP/s"}}}))
        return 0
    if args.scenario:
        return scenario(args.scenario, args.layers, args.dtype)
    sizes = SHAPES[args.shape]
    full_layers = sizes["layers_full"]
    args.layers = args.layers or full_layers

    import torch

    from tinyserve_llm_amd.config import LlamaConfig, RopeScaling
    from tinyserve_llm_amd.engine.llm import LLM, CacheConfig
    from tinyserve_llm_amd.engine.loading import random_model
    from tinyserve_llm_amd.engine.scheduler import SchedulerConfig
    from tinyserve_llm_amd.engine.sequence import SamplingParams

    config = LlamaConfig(num_hidden_layers=args.layers, rope_scaling=RopeScaling(**{**ROPE, "factor": sizes["rope_factor"]}),
                         **sizes["shape"])
    dtype = torch.bfloat16 if args.dtype == "bf16" else torch.float32
    itemsize = 2 if args.dtype == "bf16" else 4
    model = random_model(config, 0, dtype, "cuda:0")
    rng = random.Random(0)

    c = config
    layer_weights = (c.q_size + 2 * c.kv_size) * c.hidden_size + c.hidden_size * c.q_size \
        + 3 * c.intermediate_size * c.hidden_size
    weight_bytes = (args.layers * layer_weights + c.vocab_size * c.hidden_size) * itemsize   # the head; the embedding reads rows
    kv_bytes_per_token = 2 * args.layers * c.kv_size * itemsize

    prompt_len = args.context
    max_model_len = max(MAX_MODEL_LEN, prompt_len + 1024)

    def engine(batch: int, steps: int) -> LLM:
        pages = batch * -(-max_model_len // PAGE) + 2
        sc = SchedulerConfig(max_model_len=max_model_len, max_num_seqs=max(batch, 1),
                             max_num_batched_tokens=max(prompt_len, batch + 1) + batch, watermark=0.0)
        return LLM(None, sc, CacheConfig(block_size=PAGE, caching=False), dtype=dtype, num_blocks=pages, seed=0,
                   model=model)

    def decode(batch: int, steps: int, warmup: int, classes: bool = False):
        """(seconds for `steps` decode steps, mean context length over them); with `classes`, the
        kernel classes of one such step instead."""
        llm = engine(batch, steps + warmup)
        sp = SamplingParams(max_tokens=max_model_len - prompt_len, temperature=0.0, ignore_eos=True)
        for _ in range(batch):
            llm.add_request([rng.randrange(c.vocab_size) for _ in range(prompt_len)], sp)
        while any(s.in_prefill or not s.output_token_ids for s in llm.scheduler.running + llm.scheduler.waiting):
            llm.step()
        for _ in range(warmup):
            llm.step()
        assert len(llm.scheduler.running) == batch and not llm.scheduler.waiting
        if classes:
            return kernel_classes(llm, c, batch)
        ctx0 = llm.scheduler.running[0].num_tokens
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            llm.step()
        torch.cuda.synchronize()
        seconds = time.perf_counter() - t0
        assert all(r.num_tokens == batch for r in llm.steps[-steps:])
        return seconds, ctx0 + (steps - 1) / 2

    def prefill(reps: int = 3) -> float:
        llm = engine(1, 1)
        sp = SamplingParams(max_tokens=1, temperature=0.0, ignore_eos=True)
        times = []
        for r in range(reps + 1):
            llm.add_request([rng.randrange(c.vocab_size) for _ in range(prompt_len)], sp)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            llm.step()
            torch.cuda.synchronize()
            if r:
                times.append(time.perf_counter() - t0)
            assert not llm.scheduler.has_unfinished()
        return min(times)

    def prefill_record() -> dict:
        t = prefill()
        T = prompt_len
        linear_flops = 2 * T * args.layers * layer_weights + 2 * c.vocab_size * c.hidden_size
        attn_flops = args.layers * 4 * c.q_size * T * (T + 1) / 2
        return {"value": T / t, "tokens": T, "ms": 1e3 * t, "frac": (linear_flops + attn_flops) / t / PEAK_FLOPS[args.dtype]}

    if args.only == "prefill":
        print(json.dumps({"prefill": prefill_record()}))
        return 0
    if args.kernel_classes:
        print(json.dumps({"kernel_classes": decode(args.batch, 1, args.warmup, classes=True),
                          "config": {"model": sizes["model"], "layers": args.layers, "context": prompt_len, "dtype": args.dtype}}))
        return 0

    from tinyserve_llm_amd.ops import hip
    measured = hip.measure_peaks()       # what this box gives a kernel that only reads, and a loop of matrix instructions
    read_peak = measured["read_GBps"] * 1e9
    mfma_peak = measured["mfma_bf16_TFLOPs"] * 1e12 if args.dtype == "bf16" else None

    seconds, mean_ctx = decode(args.batch, args.steps, args.warmup)
    value = args.batch * args.steps / seconds
    step_bytes = weight_bytes + args.batch * mean_ctx * kv_bytes_per_token
    achieved = step_bytes / (seconds / args.steps)
    record = {
        "metric": f"decode tok/s at batch {args.batch} ({sizes['model']}, {prompt_len:,}-token contexts)",
        "value": value, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": 1e3 * seconds / args.steps, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": args.dtype, "data": "synthetic uniform token ids, random weights N(0,0.02)",
        "config": {"model": sizes["model"], "layers": args.layers, "layers_full": full_layers,
                   "hidden": c.hidden_size, "heads": c.num_attention_heads, "kv_heads": c.num_key_value_heads,
                   "head_dim": c.head_dim, "intermediate": c.intermediate_size, "vocab": c.vocab_size,
                   "global_batch": args.batch, "prompt_len": prompt_len, "seq_len": max_model_len,
                   "page_size": PAGE, "parallelism": "single-gpu"},
        "roofline": {"bound": "hbm", "achieved": achieved / 1e9, "peak": HBM_BYTES_PER_S / 1e9, "unit": "GB/s",
                     "frac": achieved / HBM_BYTES_PER_S, "measured_peak": read_peak / 1e9,
                     "frac_of_measured": achieved / read_peak},
    }
    if not args.no_prefill:
        record["prefill"] = prefill_record()
        if mfma_peak:
            record["prefill"]["measured_peak_tflops"] = mfma_peak / 1e12
            record["prefill"]["frac_of_measured"] = record["prefill"]["frac"] * PEAK_FLOPS[args.dtype] / mfma_peak
    points, detail = {}, {}
    for b in [int(x) for x in args.points.split(",") if x.strip()]:
        k = max(16, min(args.steps, 64))
        s, ctx = decode(b, k, 4)
        points[f"decode_b{b}"] = b * k / s
        rate = (weight_bytes + b * ctx * kv_bytes_per_token) / (s / k)
        detail[f"decode_b{b}"] = {"tok_s": b * k / s, "ms_per_step": 1e3 * s / k, "frac": rate / HBM_BYTES_PER_S,
                                  "frac_of_measured": rate / read_peak}
    if points:
        record["points"] = points
        record["points_detail"] = detail
    print(json.dumps(record))
    return 0


if __name__ == "__main__":
    sys.exit(main())

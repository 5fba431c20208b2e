"""Decode and prefill throughput of the Llama-3.2-1B shape with random weights on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A "step" is one decode step of the whole engine (scheduler, step function, kernels, sampling) at
batch 8 with 2,048-token contexts that grow while decoding. Prints ONE JSON line. The same line
carries the 2,048-token prefill, the decode step's HBM roofline, and decode at batch 1 and 64.
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

FULL_LAYERS = 16
SHAPE = dict(vocab_size=128256, hidden_size=2048, intermediate_size=8192, num_attention_heads=32,
             num_key_value_heads=8, head_dim=64, max_position_embeddings=131072, rms_norm_eps=1e-5,
             rope_theta=500000.0, tie_word_embeddings=True)
ROPE = dict(factor=32.0, low_freq_factor=1.0, high_freq_factor=4.0, original_max_position_embeddings=8192)
PROMPT_LEN, MAX_MODEL_LEN, PAGE = 2048, 4096, 256


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=FULL_LAYERS)
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--points", default="1,64", help="further decode batch sizes (comma-separated; '' for none)")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--only", default="all", choices=["all", "prefill"],
                    help="'prefill': time the 2,048-token prefill alone and print its record (for profiling)")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported by this engine")
        return 2

    import torch

    from tinyserve_llm_amd.config import LlamaConfig, RopeScaling
    from tinyserve_llm_amd.engine.llm import LLM, CacheConfig
    from tinyserve_llm_amd.engine.loading import random_model
    from tinyserve_llm_amd.engine.scheduler import SchedulerConfig
    from tinyserve_llm_amd.engine.sequence import SamplingParams

    config = LlamaConfig(num_hidden_layers=args.layers, rope_scaling=RopeScaling(**ROPE), **SHAPE)
    dtype = torch.bfloat16 if args.dtype == "bf16" else torch.float32
    itemsize = 2 if args.dtype == "bf16" else 4
    model = random_model(config, 0, dtype, "cuda:0")
    rng = random.Random(0)

    c = config
    layer_weights = (c.q_size + 2 * c.kv_size) * c.hidden_size + c.hidden_size * c.q_size \
        + 3 * c.intermediate_size * c.hidden_size
    weight_bytes = (args.layers * layer_weights + c.vocab_size * c.hidden_size) * itemsize
    kv_bytes_per_token = 2 * args.layers * c.kv_size * itemsize

    def engine(batch: int, steps: int) -> LLM:
        pages = batch * (MAX_MODEL_LEN // PAGE) + 2
        sc = SchedulerConfig(max_model_len=MAX_MODEL_LEN, max_num_seqs=max(batch, 1),
                             max_num_batched_tokens=max(PROMPT_LEN, batch + 1) + batch, watermark=0.0)
        return LLM(None, sc, CacheConfig(block_size=PAGE, caching=False), dtype=dtype, num_blocks=pages, seed=0,
                   model=model)

    def decode(batch: int, steps: int, warmup: int) -> tuple[float, float]:
        """(seconds for `steps` decode steps, mean context length over them)."""
        llm = engine(batch, steps + warmup)
        sp = SamplingParams(max_tokens=MAX_MODEL_LEN - PROMPT_LEN, temperature=0.0, ignore_eos=True)
        for _ in range(batch):
            llm.add_request([rng.randrange(c.vocab_size) for _ in range(PROMPT_LEN)], sp)
        while any(s.in_prefill or not s.output_token_ids for s in llm.scheduler.running + llm.scheduler.waiting):
            llm.step()
        for _ in range(warmup):
            llm.step()
        assert len(llm.scheduler.running) == batch and not llm.scheduler.waiting
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
            llm.add_request([rng.randrange(c.vocab_size) for _ in range(PROMPT_LEN)], sp)
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
        T = PROMPT_LEN
        linear_flops = 2 * T * args.layers * layer_weights + 2 * c.vocab_size * c.hidden_size
        attn_flops = args.layers * 4 * c.q_size * T * (T + 1) / 2
        return {"value": T / t, "tokens": T, "ms": 1e3 * t, "frac": (linear_flops + attn_flops) / t / PEAK_FLOPS[args.dtype]}

    if args.only == "prefill":
        print(json.dumps({"prefill": prefill_record()}))
        return 0

    seconds, mean_ctx = decode(args.batch, args.steps, args.warmup)
    value = args.batch * args.steps / seconds
    step_bytes = weight_bytes + args.batch * mean_ctx * kv_bytes_per_token
    achieved = step_bytes / (seconds / args.steps)
    record = {
        "metric": "decode tok/s at batch 8 (Llama-3.2-1B shape, 2,048-token contexts)",
        "value": value, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": 1e3 * seconds / args.steps, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": args.dtype, "data": "synthetic uniform token ids, random weights N(0,0.02)",
        "config": {"model": "llama-3.2-1b-shape", "layers": args.layers, "layers_full": FULL_LAYERS,
                   "hidden": c.hidden_size, "heads": c.num_attention_heads, "kv_heads": c.num_key_value_heads,
                   "head_dim": c.head_dim, "intermediate": c.intermediate_size, "vocab": c.vocab_size,
                   "global_batch": args.batch, "prompt_len": PROMPT_LEN, "seq_len": MAX_MODEL_LEN,
                   "page_size": PAGE, "parallelism": "single-gpu"},
        "roofline": {"bound": "hbm", "achieved": achieved / 1e9, "peak": HBM_BYTES_PER_S / 1e9, "unit": "GB/s",
                     "frac": achieved / HBM_BYTES_PER_S},
    }
    if not args.no_prefill:
        record["prefill"] = prefill_record()
    points = {}
    for b in [int(x) for x in args.points.split(",") if x.strip()]:
        k = max(16, min(args.steps, 64))
        s, _ = decode(b, k, 4)
        points[f"decode_b{b}"] = b * k / s
    if points:
        record["points"] = points
    print(json.dumps(record))
    return 0


if __name__ == "__main__":
    sys.exit(main())

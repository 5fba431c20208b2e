"""Command line of the engine, in the manner of the reference's benchmark modules
(benchmarks/run_ours.py:59-130: argparse, progress lines, one JSON record):

    python -m tinyserve_llm_amd.generate --model DIR --prompt-ids 5,17,3 --prompt-ids 9,9 \\
        --max-tokens 16 --temperature 0 --out result.json
    python -m tinyserve_llm_amd.generate --random-config config.json --random-seed 0 --prompt-lengths 17,33

Prompts are token ids (`--prompt-ids`, repeatable), files of them (`--prompts-file`, one JSON list
per line), seeded random ids of given lengths (`--prompt-lengths`), or text if the model folder
holds a tokenizer (`--prompt`).
"""

from __future__ import annotations

import argparse
import json
import random
import sys
import time
from dataclasses import asdict

import torch


def parse_args(argv=None) -> argparse.Namespace:
    p = argparse.ArgumentParser(prog="python -m tinyserve_llm_amd.generate")
    p.add_argument("--model", help="folder with config.json and model*.safetensors")
    p.add_argument("--random-config", help="a config.json to run with random weights instead of --model")
    p.add_argument("--random-seed", type=int, default=0, help="seed of the random weights")
    p.add_argument("--prompt", action="append", default=[], help="text prompt (needs a tokenizer in --model)")
    p.add_argument("--prompt-ids", action="append", default=[], help="comma-separated token ids; repeatable")
    p.add_argument("--prompts-file", help="file with one JSON list of token ids per line")
    p.add_argument("--prompt-lengths", help="comma-separated lengths of seeded uniform random prompts")
    p.add_argument("--max-tokens", type=int, default=256)
    p.add_argument("--temperature", type=float, default=0.6)
    p.add_argument("--n", type=int, default=1, help="parallel samples per prompt")
    p.add_argument("--ignore-eos", action="store_true")
    p.add_argument("--seed", type=int, default=0)
    p.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    p.add_argument("--caching", choices=["on", "off"], default="on")
    p.add_argument("--block-size", type=int, default=256)
    p.add_argument("--num-blocks", type=int, default=None, help="pages of the KV cache; default: from free memory")
    p.add_argument("--gpu-memory-utilization", type=float, default=0.9)
    p.add_argument("--max-model-len", type=int, default=4096)
    p.add_argument("--max-num-seqs", type=int, default=512)
    p.add_argument("--max-num-batched-tokens", type=int, default=16384)
    p.add_argument("--max-prefill-chunk", type=int, default=0)
    p.add_argument("--device", default="cuda")
    p.add_argument("--many-rows-products", choices=["library", "tiled"], default="library",
                   help="bfloat16 products of many rows: the vendor's matrix library, or the engine's own tiled kernel (slower)")
    p.add_argument("--no-library-timing", action="store_true",
                   help="keep the matrix library's first candidate for every shape instead of timing candidates: "
                        "two runs then round every product alike")
    p.add_argument("--out", help="write the JSON record here as well as printing a summary")
    return p.parse_args(argv)


def _library_choices() -> list:
    """Which of the matrix library's algorithms served which shape in this run (bfloat16 roundings
    follow from them)."""
    from tinyserve_llm_amd.ops import hip
    return hip.library_choices()


def main(argv=None) -> int:
    args = parse_args(argv)
    if bool(args.model) == bool(args.random_config):
        print("give exactly one of --model and --random-config", file=sys.stderr)
        return 2
    from tinyserve_llm_amd.engine.llm import LLM, CacheConfig
    from tinyserve_llm_amd.engine.scheduler import SchedulerConfig
    from tinyserve_llm_amd.engine.sequence import SamplingParams
    from tinyserve_llm_amd.models.registry import resolve

    random_weights = None
    if args.random_config:
        with open(args.random_config) as f:
            raw = json.load(f)
        random_weights = (resolve(raw).config_from_dict(raw), args.random_seed)
    sc = SchedulerConfig(max_model_len=args.max_model_len, max_num_seqs=args.max_num_seqs,
                         max_num_batched_tokens=args.max_num_batched_tokens, max_prefill_chunk=args.max_prefill_chunk)
    cc = CacheConfig(block_size=args.block_size, caching=args.caching == "on", device=args.device)
    if args.many_rows_products != "library":
        from tinyserve_llm_amd.ops import hip
        hip.many_rows_products(args.many_rows_products)
    llm = LLM(args.model, sc, cc, dtype=args.dtype, num_blocks=args.num_blocks,
              gpu_memory_utilization=args.gpu_memory_utilization, seed=args.seed, random_weights=random_weights,
              time_library=not args.no_library_timing)
    vocab = llm.model.spec.vocab_size
    prompts: list = list(args.prompt)
    prompts += [[int(t) for t in ids.split(",") if t.strip()] for ids in args.prompt_ids]
    if args.prompts_file:
        with open(args.prompts_file) as f:
            prompts += [json.loads(line) for line in f if line.strip()]
    if args.prompt_lengths:
        rng = random.Random(args.seed)
        prompts += [[rng.randrange(vocab) for _ in range(int(n))] for n in args.prompt_lengths.split(",")]
    if not prompts:
        print("no prompts: use --prompt-ids, --prompts-file, --prompt-lengths or --prompt", file=sys.stderr)
        return 2
    print(f"{len(prompts)} prompts; KV {llm.manager.num_blocks} blocks of {args.block_size} tokens; "
          f"dtype {args.dtype}", flush=True)
    params = SamplingParams(max_tokens=args.max_tokens, temperature=args.temperature, n=args.n,
                            ignore_eos=args.ignore_eos)
    started = time.time()
    t0 = time.perf_counter()
    results = llm.generate(prompts, params)
    seconds = time.perf_counter() - t0
    out_tokens = sum(len(t) for r in results for t in r.token_ids)
    for r in results:
        for k, toks in enumerate(r.token_ids):
            shown = r.texts[k] if r.texts else " ".join(map(str, toks))
            print(f"request {r.request_id} sample {k} [{r.finish_reasons[k]}]: {shown}", flush=True)
    stats = llm.scheduler.stats()
    record = {
        "engine": "tinyserve_llm_amd", "model": args.model or args.random_config, "dtype": args.dtype,
        "num_blocks": llm.manager.num_blocks, "block_size": args.block_size, "caching": args.caching,
        "temperature": args.temperature, "seed": args.seed, "n": args.n, "max_tokens": args.max_tokens,
        "device": torch.cuda.get_device_name(), "torch": torch.__version__, "started": started,
        "seconds": seconds, "output_tokens": out_tokens, "output_tokens_per_second": out_tokens / seconds,
        "steps": len(llm.steps), "library_choices": _library_choices(), "scheduler_stats": asdict(stats), "cache_stats": asdict(llm.manager.stats()),
        "completions": [{"request_id": r.request_id, "prompt_token_ids": r.prompt_token_ids, "token_ids": r.token_ids,
                         "texts": r.texts, "finish_reasons": r.finish_reasons} for r in results],
    }
    if args.out:
        with open(args.out, "w") as f:
            json.dump(record, f)
    print(f"{out_tokens} output tokens in {seconds:.2f} s ({out_tokens / seconds:,.0f} tok/s), "
          f"{stats.prefill_tokens:,} prefilled, {stats.cached_tokens:,} from cache, {stats.preemptions} preempted"
          + (f"; wrote {args.out}" if args.out else ""), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())

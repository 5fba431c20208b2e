"""Trace replay: given token ids go through the model step by step and logits are written out.
Nothing is sampled. It drives the same model, step function, cache manager and kernels that
generation uses; the reference has nothing of the kind (its nearest code drives
schedule/prepare/forward/postprocess by hand in tests/test_gpu.py:89-110).

Steps arrive as JSON lines:
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
For a step in which something is wanted, `<out>/<step>.f32` holds the logits at the wanted places
in the order of the entries and of `want`, little-endian float32 [wanted, vocab].
"""

from __future__ import annotations

import argparse
import json
import os
import sys

import numpy as np
import torch

from tinyserve_llm_amd.engine.interface import build_cache
from tinyserve_llm_amd.engine.loading import as_dtype, load_model
from tinyserve_llm_amd.engine.runner import ModelRunner, StepEntry

REPLAY_PAGE_SIZE = 64
MAX_LIVE = 16


class Replay:
    def __init__(self, model_dir: str, dtype: str, max_tokens: int, device: str = "cuda:0",
                 page_size: int = REPLAY_PAGE_SIZE) -> None:
        self.model, self.config = load_model(model_dir, dtype, device)
        num_pages = max(1, -(-max_tokens // page_size))
        # replay runs exactly the tokens it is given, so nothing is ever taken from a prefix cache
        self.storage, self.manager = build_cache(self.model, num_pages, page_size, as_dtype(dtype), device,
                                                 num_state_slots=MAX_LIVE, caching=False)
        self.runner = ModelRunner(self.model, self.storage, self.manager)
        self.ids: dict[str, int] = {}
        self.lengths: dict[int, int] = {}
        self._next = 0

    def step(self, entries: list[dict], end: list[str]) -> torch.Tensor:
        batch: list[StepEntry] = []
        for e in entries:
            name, tokens = str(e["id"]), [int(t) for t in e["tokens"]]
            if name not in self.ids:
                seq = self.ids[name] = self._next
                self._next += 1
                if self.manager.allocate(seq, tokens) is None:
                    raise RuntimeError(f"request {name!r}: no pages left for {len(tokens)} tokens "
                                       f"({self.manager.num_available_blocks()} pages of {self.storage.page_size} free)")
                self.lengths[seq] = 0
            else:
                seq = self.ids[name]
                if not self.manager.can_append(seq, len(tokens)):
                    raise RuntimeError(f"request {name!r}: no pages left for {len(tokens)} more tokens")
                self.manager.append_slots(seq, tokens)
            batch.append(StepEntry(seq, tokens, self.lengths[seq], [int(w) for w in e.get("want", [])]))
        logits = self.runner.step(batch) if batch else torch.empty((0, self.model.spec.vocab_size))
        for e in batch:
            self.manager.commit(e.seq_id, len(e.tokens))
            self.lengths[e.seq_id] += len(e.tokens)
        for name in end:
            seq = self.ids.pop(str(name), None)
            if seq is not None:
                self.manager.release(seq)
                del self.lengths[seq]
        return logits


def main(argv: list[str] | None = None) -> int:
    parser = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    parser.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    parser.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    parser.add_argument("--out", required=True, help="folder for <step>.f32 files")
    parser.add_argument("--max-tokens", type=int, required=True,
                        help="most tokens live requests hold at any time (each rounded up to a page of 64)")
    parser.add_argument("--device", default="cuda:0")
    args = parser.parse_args(argv)
    os.makedirs(args.out, exist_ok=True)
    replay = Replay(args.model, args.dtype, args.max_tokens, args.device)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        record = json.loads(line)
        step = record["step"]
        logits = replay.step(record.get("entries", []), record.get("end", []))
        if logits.shape[0]:
            np.ascontiguousarray(logits.cpu().numpy().astype("<f4")).tofile(os.path.join(args.out, f"{step}.f32"))
        else:
            torch.cuda.synchronize()
        print(f"done {step}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())

"""The engine loop and the Python entry point: LLM(path).generate(prompts, SamplingParams(...))
(tinyserve_llm/engine/llm_engine.py:26-185). schedule -> run the step -> sample -> postprocess,
until nothing is waiting or running."""

from __future__ import annotations

import logging
import os
import time
from dataclasses import dataclass, replace
from typing import Literal

import torch

from tinyserve_llm_amd.cache.manager import CacheStats, KVCacheManager
from tinyserve_llm_amd.cache.storage import KVStorage, bytes_per_page
from tinyserve_llm_amd.models.decoder import DecoderModel
from tinyserve_llm_amd.engine.loading import as_dtype, load_model, random_model, require_gpu
from tinyserve_llm_amd.engine.runner import ModelRunner, StepEntry
from tinyserve_llm_amd.engine.scheduler import RequestOutput, ScheduledSeq, Scheduler, SchedulerConfig, SchedulerStats
from tinyserve_llm_amd.engine.sequence import SamplingParams
from tinyserve_llm_amd.sampling.sampler import row_key, sample

logger = logging.getLogger(__name__)


@dataclass(frozen=True)
class CacheConfig:
    block_size: int = 256
    caching: bool = True        # False: no prefix reuse; forks still share pages
    device: str = "cuda"


@dataclass
class StepRecord:
    """One engine step; the stats are running totals (subtract consecutive records)."""
    start: float
    end: float
    num_seqs: int
    num_tokens: int
    scheduler: SchedulerStats
    cache: CacheStats


@dataclass
class Completion:
    request_id: int
    prompt_token_ids: list[int]
    token_ids: list[list[int]]           # the n samples, in fork order
    texts: list[str] | None
    finish_reasons: list[Literal["eos", "length"]]
    arrival_time: float
    first_token_time: float
    finish_time: float


class LLM:
    def __init__(
            self,
            model_path: str | None,
            scheduler_config: SchedulerConfig = SchedulerConfig(),
            cache_config: CacheConfig = CacheConfig(),
            *,
            dtype: torch.dtype | str = torch.bfloat16,
            num_blocks: int | None = None,           # None: sized from free GPU memory
            gpu_memory_utilization: float = 0.9,
            seed: int | None = None,
            load_tokenizer: bool | None = None,      # None: only if the folder holds a tokenizer
            random_weights: tuple[object, int] | None = None,   # (typed configuration, seed) instead of a folder
            model: DecoderModel | None = None,       # an already bound model (shares its weights)
            decode_graphs: bool = True,              # replay decode steps from HIP graphs
    ) -> None:
        self.device = require_gpu(cache_config.device if cache_config.device != "cuda" else "cuda:0")
        self.dtype = as_dtype(dtype)
        if model is not None:
            self.model, self.config = model, None
            self.dtype = model.dtype
        elif random_weights is not None:
            self.config, weight_seed = random_weights
            self.model = random_model(self.config, weight_seed, self.dtype, self.device)
        else:
            if model_path is None:
                raise ValueError("give a model folder or random_weights=(config, seed)")
            self.model, self.config = load_model(model_path, self.dtype, self.device)
        spec = self.model.spec
        if scheduler_config.max_model_len > spec.max_position:
            raise ValueError(f"max_model_len {scheduler_config.max_model_len} exceeds the model's "
                             f"{spec.max_position} positions")
        self.tokenizer = None
        if load_tokenizer is None:
            load_tokenizer = model_path is not None and any(
                os.path.exists(os.path.join(model_path, f)) for f in ("tokenizer.json", "tokenizer.model"))
        if load_tokenizer:
            from transformers import AutoTokenizer       # text in and out only; no model code
            self.tokenizer = AutoTokenizer.from_pretrained(model_path)
        if scheduler_config.eos_token_id == -1:
            scheduler_config = replace(scheduler_config, eos_token_id=self._eos_token_id())
        self.seed = 0 if seed is None else seed
        cache_plan, state_plan = self.model.cache_plan(), self.model.state_plan()
        if num_blocks is None:
            num_blocks = self._size_from_free_memory(scheduler_config, cache_config, gpu_memory_utilization)
        self.storage = KVStorage(cache_plan, state_plan, num_blocks, cache_config.block_size, self.dtype, self.device,
                                 num_state_slots=scheduler_config.max_num_seqs)
        self.manager = KVCacheManager(self.storage, caching=cache_config.caching)
        self.scheduler = Scheduler(scheduler_config, self.manager)
        self.runner = ModelRunner(self.model, self.storage, self.manager)
        if decode_graphs:
            self.runner.enable_decode_graphs(scheduler_config.max_model_len, scheduler_config.max_num_seqs, self.seed)
        self.steps: list[StepRecord] = []
        logger.info("KV cache: %d blocks of %d tokens", num_blocks, cache_config.block_size)

    def _eos_token_id(self) -> int:
        if self.tokenizer is not None and self.tokenizer.eos_token_id is not None:
            return self.tokenizer.eos_token_id
        return self.model.spec.eos_token_id

    def _size_from_free_memory(self, sc: SchedulerConfig, cc: CacheConfig, utilisation: float) -> int:
        """Pages from what the GPU has left under the utilisation limit, after setting aside the
        activations of a worst-case step (llm_engine.py:112-140 measures them with a trial step;
        here they are bounded from the model's widths)."""
        free, total = torch.cuda.mem_get_info(self.device)
        widest = max([self.model.spec.hidden_size] + [p.shape[0] for n, p in self.model.param_specs().items()
                                                        if n.startswith("layers.") and len(p.shape) == 2])
        act = sc.max_num_batched_tokens * widest * 4 * 6 + sc.max_num_seqs * self.model.spec.vocab_size * 4 * 2
        budget = total * utilisation - (total - free) - act
        per_page = max(1, bytes_per_page(self.model.cache_plan(), cc.block_size, self.dtype))
        pages = int(budget // per_page)
        most_useful = sc.max_num_seqs * (-(-sc.max_model_len // cc.block_size) + 1) + 8
        pages = min(pages, most_useful)
        if pages <= 0:
            raise RuntimeError("no memory left for the KV cache; lower max_num_batched_tokens or raise utilisation")
        return pages

    # ---- requests ---------------------------------------------------------------------------
    def add_request(self, prompt: str | list[int], params: SamplingParams, arrival_time: float | None = None) -> int:
        if isinstance(prompt, str):
            if self.tokenizer is None:
                raise ValueError("a text prompt needs load_tokenizer=True; pass token ids otherwise")
            token_ids = self.tokenizer.encode(prompt)
        else:
            token_ids = list(prompt)
        vocab = self.model.spec.vocab_size
        if any(not 0 <= t < vocab for t in token_ids):
            raise ValueError(f"prompt holds token ids outside the vocabulary of {vocab}")
        return self.scheduler.add_request(token_ids, params, time.perf_counter() if arrival_time is None else arrival_time)

    def _run(self, batch: list[ScheduledSeq]) -> list[list[int]]:
        """One forward pass and the draws; one host sync (model_runner.py:120-133)."""
        entries, temps, keys, owners = [], [], [], []
        for seq, tokens, num_samples, start in batch:
            entries.append(StepEntry(seq.seq_id, tokens, start, [len(tokens) - 1] if num_samples else []))
        if all(b.num_samples == 1 for b in batch):
            # one draw per entry: the step function draws too (decode steps replay one graph for both)
            for seq, tokens, num_samples, start in batch:
                temps.append(seq.params.temperature)
                keys.append(row_key(seq.request_id, seq.sample_index, len(seq.output_token_ids)))
            return [[t] for t in self.runner.step_sample(entries, temps, keys, self.seed).tolist()]
        logits = self.runner.step(entries)
        row = 0
        rows: list[int] = []
        for seq, tokens, num_samples, start in batch:
            for k in range(num_samples):
                # the k-th sample of a group's first token; later tokens belong to seq.sample_index
                index = k if num_samples > 1 else seq.sample_index
                temps.append(seq.params.temperature)
                keys.append(row_key(seq.request_id, index, len(seq.output_token_ids)))
                rows.append(row)
            if num_samples:
                row += 1
            owners.append(num_samples)
        if not rows:
            torch.cuda.current_stream().synchronize()
            return [[] for _ in batch]
        picked = logits if rows == list(range(logits.shape[0])) else logits[torch.tensor(rows, device=logits.device)]
        tokens = sample(picked, temps, keys, self.seed).tolist()
        out, i = [], 0
        for n in owners:
            out.append(tokens[i:i + n])
            i += n
        return out

    def step(self) -> list[RequestOutput]:
        start = time.perf_counter()
        batch = self.scheduler.schedule(start)
        if not batch:
            raise RuntimeError("the scheduler produced an empty step")
        sampled = self._run(batch)
        end = time.perf_counter()
        outputs = self.scheduler.postprocess(batch, sampled, end)
        self.steps.append(StepRecord(start, end, len(batch), sum(len(b.token_ids) for b in batch),
                                     self.scheduler.stats(), self.manager.stats()))
        return outputs

    def generate(self, prompts: list[str] | list[list[int]],
                 params: SamplingParams | list[SamplingParams] = SamplingParams()) -> list[Completion]:
        """Runs the prompts to completion; results in prompt order."""
        params = params if isinstance(params, list) else [params] * len(prompts)
        order = [self.add_request(p, sp) for p, sp in zip(prompts, params, strict=True)]
        done: dict[int, RequestOutput] = {}
        while self.scheduler.has_unfinished():
            for output in self.step():
                done[output.request_id] = output
        return [self._completion(done[r]) for r in order]

    def _completion(self, output: RequestOutput) -> Completion:
        seqs = output.sequences
        token_ids = [list(s.output_token_ids) for s in seqs]
        texts = None
        if self.tokenizer is not None:
            texts = [self.tokenizer.decode(t, skip_special_tokens=True) for t in token_ids]
        return Completion(
            request_id=output.request_id, prompt_token_ids=list(seqs[0].prompt_token_ids), token_ids=token_ids,
            texts=texts, finish_reasons=[s.finish_reason for s in seqs], arrival_time=seqs[0].arrival_time,
            first_token_time=min(s.first_token_time for s in seqs), finish_time=max(s.finish_time for s in seqs))

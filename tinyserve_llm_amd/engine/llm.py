"""The engine loop and the Python entry point: LLM(path).generate(prompts, SamplingParams(...))
(tinyserve_llm/engine/llm_engine.py:26-185). schedule -> run the step -> sample -> postprocess,
until nothing is waiting or running. Decode steps overlap with the host: while the device runs
one, the next is already scheduled and packed (see `LLM.step`)."""

from __future__ import annotations

import logging
import os
import time
from dataclasses import dataclass, replace
from typing import Literal, Sequence

import torch

from tinyserve_llm_amd.engine.interface import CacheConfig, CacheStats, build_cache, bytes_per_page
from tinyserve_llm_amd.engine.loading import as_dtype, load_model, random_model, require_gpu
from tinyserve_llm_amd.models.decoder import DecoderModel
from tinyserve_llm_amd.engine.runner import DecodeGraphs, ModelRunner, StepEntry
from tinyserve_llm_amd.engine.scheduler import (PENDING, RequestOutput, ScheduledSeq, Scheduler, SchedulerConfig,
                                                SchedulerStats)
from tinyserve_llm_amd.engine.sequence import SamplingParams
from tinyserve_llm_amd.sampling.sampler import row_key, sample

logger = logging.getLogger(__name__)


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

    @classmethod
    def of(cls, output: RequestOutput, tokenizer=None) -> "Completion":
        """A finished request as its caller sees it: the samples' tokens in fork order (and their
        text, if there is a tokenizer), the time of the first token of any sample and of the last
        sample's end (llm_engine.py:170-185)."""
        first = output.sequences[0]
        samples = [list(seq.output_token_ids) for seq in output.sequences]
        return cls(
            output.request_id, list(first.prompt_token_ids), samples,
            None if tokenizer is None else [tokenizer.decode(ids, skip_special_tokens=True) for ids in samples],
            [seq.finish_reason for seq in output.sequences], first.arrival_time,
            min(seq.first_token_time for seq in output.sequences),
            max(seq.finish_time for seq in output.sequences))


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
            run_ahead: bool = True,                  # schedule and pack the next decode step while this one runs
            keep_streaming_copies: bool | None = None,   # layer weights once more in the decode kernels' order; None: if memory is ample
            max_decode_graphs: int = DecodeGraphs.MAX_GRAPHS,         # recorded decode steps kept at most (least recently replayed out),
            decode_graph_memory: int = DecodeGraphs.MEMORY_BUDGET,    # and the bytes their own buffers may take
            record_decode_steps: Sequence[int | tuple[int, int]] = (),   # batch sizes (or (batch size, context)) to record now, not at first use
            time_library: bool = True,               # time the matrix library's candidates when a step is recorded (faster; roundings may differ between runs)
    ) -> None:
        self.device = require_gpu(cache_config.device if cache_config.device != "cuda" else "cuda:0")
        self.dtype = as_dtype(dtype)
        if model is not None:
            self.model, self.config = model, None
            self.dtype = model.dtype
        elif random_weights is not None:
            self.config, weight_seed = random_weights
            self.model = random_model(self.config, weight_seed, self.dtype, self.device, keep_streaming_copies)
        else:
            if model_path is None:
                raise ValueError("give a model folder or random_weights=(config, seed)")
            self.model, self.config = load_model(model_path, self.dtype, self.device, keep_streaming_copies)
        spec = self.model.spec
        if spec.max_position is not None and scheduler_config.max_model_len > spec.max_position:
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
        graphs_on = decode_graphs and self.model.graph_safe()
        if not time_library:
            from tinyserve_llm_amd.ops import hip
            hip.library_timing(False)                # (for the process: also the choice among three for steps of many rows)
        if num_blocks is None:
            num_blocks = self._size_from_free_memory(scheduler_config, cache_config, gpu_memory_utilization,
                                                     decode_graph_memory if graphs_on else 0)
        self.storage, self.manager = build_cache(self.model, num_blocks, cache_config.block_size, self.dtype, self.device,
                                                 num_state_slots=scheduler_config.max_num_seqs,
                                                 caching=cache_config.caching)
        self.scheduler = Scheduler(scheduler_config, self.manager)
        self.runner = ModelRunner(self.model, self.storage, self.manager)
        if graphs_on:
            self.runner.enable_decode_graphs(scheduler_config.max_model_len, scheduler_config.max_num_seqs, self.seed,
                                             max_graphs=max_decode_graphs, memory_budget=decode_graph_memory,
                                             time_library=time_library)
            for wanted in record_decode_steps:
                batch, context = wanted if isinstance(wanted, tuple) else (wanted, scheduler_config.max_model_len)
                self.runner.graphs.record(batch, context)
        self.run_ahead = run_ahead
        self._ahead: tuple | None = None             # (what is left of the step scheduled ahead, its launch or None, its rows)
        self.steps: list[StepRecord] = []
        logger.info("KV cache: %d blocks of %d tokens", num_blocks, cache_config.block_size)

    def _eos_token_id(self) -> int:
        if self.tokenizer is not None and self.tokenizer.eos_token_id is not None:
            return self.tokenizer.eos_token_id
        return self.model.spec.eos_token_id

    def _size_from_free_memory(self, sc: SchedulerConfig, cc: CacheConfig, utilisation: float, graph_memory: int) -> int:
        """Pages from what the GPU has left under the utilisation limit, after setting aside what is
        allocated later: the activations of a worst-case step (llm_engine.py:112-140 measures them
        with a trial step; here the parts say how wide they get), the matrix library's workspace and
        the buffer its timing sweeps, and the recorded decode steps' own buffers (`graph_memory`,
        which `DecodeGraphs` holds itself to)."""
        from tinyserve_llm_amd.ops import hip
        free, total = torch.cuda.mem_get_info(self.device)
        widest = self.model.widest_activation()
        act = sc.max_num_batched_tokens * widest * 4 * 6 + sc.max_num_seqs * self.model.spec.vocab_size * 4 * 2
        later = act + graph_memory + hip.LIBRARY_WORKSPACE_BYTES + hip.LIBRARY_TUNING_SWEEP_BYTES
        budget = total * utilisation - (total - free) - later
        per_page = max(1, bytes_per_page(self.model, cc.block_size, self.dtype))
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

    def _draws(self, batch: list[ScheduledSeq]) -> tuple[list[float], list[int]]:
        """Temperature and key of the one draw of every entry (a key names request, sample and
        output position; a placeholder output already counts as the token it stands for)."""
        temps = [b.seq.params.temperature for b in batch]
        keys = [row_key(b.seq.request_id, b.seq.sample_index, len(b.seq.output_token_ids)) for b in batch]
        return temps, keys

    def _launch(self, batch: list[ScheduledSeq]) -> tuple:
        """Starts one forward pass and the draws on the device (model_runner.py:120-133); `_finish`
        waits for them."""
        entries = [StepEntry(seq.seq_id, tokens, start, [len(tokens) - 1] if num_samples else [])
                   for seq, tokens, num_samples, start in batch]
        if all(b.num_samples == 1 for b in batch):
            # one draw per entry: the step function draws too (decode steps replay one graph for both)
            temps, keys = self._draws(batch)
            return self.runner.step_sample(entries, temps, keys, self.seed), None
        logits = self.runner.step(entries)
        temps, keys, owners, rows = [], [], [], []
        row = 0
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
            return None, owners
        return sample(logits, temps, keys, self.seed, None if rows == list(range(logits.shape[0])) else rows), owners

    def _finish(self, launched: tuple) -> list[list[int]]:
        """Waits for a launched step; the one host sync of a step. Tokens per entry."""
        drawn, owners = launched
        if drawn is None:
            torch.cuda.current_stream().synchronize()
            return [[] for _ in owners]
        tokens = drawn.tolist()
        if owners is None:
            return [[t] for t in tokens]
        out, i = [], 0
        for n in owners:
            out.append(tokens[i:i + n])
            i += n
        return out

    def _launch_ahead(self, ahead: list[ScheduledSeq], launched: tuple, order: list[int]) -> tuple | None:
        """Packs and starts the next step while the device runs this one, if it is one of decodes
        only that the decode graphs take. Its entries whose token is still a placeholder take it on
        the device from what the running step draws (`order`: the sequence of each of its rows), so
        neither step waits for the host. None if the step has to be started the plain way."""
        drawn, owners = launched
        if not ahead or drawn is None or owners is not None or not self.scheduler.decodes_only(ahead):
            return None
        row = {seq_id: k for k, seq_id in enumerate(order)}
        entries = [StepEntry(b.seq.seq_id, [0 if t == PENDING else t for t in b.token_ids], b.start, [0]) for b in ahead]
        feed = [row[b.seq.seq_id] if b.token_ids[0] == PENDING else -1 for b in ahead]
        temps, keys = self._draws(ahead)
        prepared = self.runner.prepare_decode(entries, temps, keys, self.seed, feed)
        if prepared is None:
            return None
        return self.runner.launch_decode(prepared, drawn), None

    def step(self) -> list[RequestOutput]:
        """One step of the engine. A step of decodes only is closed in two halves: the slots are
        committed, the next step is scheduled, packed and started behind this one on the device
        (taking the tokens this one draws where they are, on the device), and only then are this
        step's tokens read and entered into the books. A sequence that turns out to have ended has
        a row in the step already started; that row is dropped when the step is read. Any other
        step is scheduled, run and closed in turn."""
        start = time.perf_counter()
        # (what is left of the step scheduled ahead, its launch, the sequence of each launched row)
        batch, launched, order = self._ahead if self._ahead is not None else (None, None, None)
        self._ahead = None
        if batch is None:
            batch = self.scheduler.schedule(start)
        if not batch:
            raise RuntimeError("the scheduler produced an empty step")
        if launched is None:
            launched, order = self._launch(batch), [b.seq.seq_id for b in batch]
        halves = self.run_ahead and self.scheduler.decodes_only(batch)
        early = None
        if halves:
            self.scheduler.commit_decodes(batch)
            ahead = self.scheduler.schedule(time.perf_counter()) if self.scheduler.has_unfinished() else []
            early = self._launch_ahead(ahead, launched, order)
        sampled = self._finish(launched)
        if len(order) != len(batch):            # rows of sequences that ended after the step was started
            row = {seq_id: k for k, seq_id in enumerate(order)}
            sampled = [sampled[row[b.seq.seq_id]] for b in batch]
        end = time.perf_counter()
        if halves:
            outputs, left = self.scheduler.deliver_tokens(batch, sampled, end, ahead)
            if left:
                self._ahead = (left, early, [b.seq.seq_id for b in ahead] if early is not None else None)
        else:
            outputs = self.scheduler.postprocess(batch, sampled, end)
        self.steps.append(StepRecord(start, end, len(batch), sum(len(b.token_ids) for b in batch),
                                     self.scheduler.stats(), self.manager.stats()))
        return outputs

    def generate(self, prompts: list[str] | list[list[int]],
                 params: SamplingParams | list[SamplingParams] = SamplingParams()) -> list[Completion]:
        """Queues every prompt (one `SamplingParams` for all, or one each), steps the engine until
        both queues are empty, and returns the completions in the order of the prompts
        (llm_engine.py:159-168)."""
        each = params if isinstance(params, list) else [params] * len(prompts)
        if len(each) != len(prompts):
            raise ValueError(f"{len(prompts)} prompts but {len(each)} sampling parameters")
        place = {self.add_request(prompt, sp): i for i, (prompt, sp) in enumerate(zip(prompts, each))}
        results: list[Completion | None] = [None] * len(prompts)
        while self.scheduler.has_unfinished():
            for finished in self.step():
                if finished.request_id in place:          # (requests queued through add_request run along)
                    results[place[finished.request_id]] = Completion.of(finished, self.tokenizer)
        return results

"""The step function: one batch of (request, its next tokens) through the model, from the cache,
with logits at the wanted places only (tinyserve_llm/engine/model_runner.py:43-133 packs and runs
whole prompt remainders and samples inside; here portions are first-class and logits come out).

A step's entries may be portions of prompts of any length beside single decoded tokens. Each
entry says where its tokens start; the cache manager has already reserved their slots. The step
runs only these tokens, writes their keys and values, attends over the pages, and returns float32
logits [wanted, vocab] in the order of the entries and of their `want` lists.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Protocol, Sequence

import torch

from tinyserve_llm_amd.cache.manager import FREED
from tinyserve_llm_amd.cache.storage import KVStorage
from tinyserve_llm_amd.models.decoder import DecoderModel
from tinyserve_llm_amd.parts.base import LayerMemory, StepContext


@dataclass
class StepEntry:
    seq_id: int
    tokens: Sequence[int]
    start: int                                        # position of tokens[0] in its request
    want: Sequence[int] = field(default_factory=list)  # indices into `tokens` whose logits are wanted


class TableView(Protocol):
    """Read access to the cache manager, valid between reserving a step's slots and committing."""

    def block_table(self, seq_id: int, space: int = 0) -> Sequence[int]: ...
    def state_slot(self, seq_id: int) -> int: ...


class StepError(ValueError):
    pass


class ModelRunner:
    def __init__(self, model: DecoderModel, storage: KVStorage, view: TableView) -> None:
        self.model = model
        self.storage = storage
        self.view = view
        self.device = storage.device
        self.memory: list[LayerMemory] = []
        for i, run in enumerate(model.spec.order):
            mem = LayerMemory(store=run.store, state=storage.state(i))
            owner = i if run.cache is None else run.cache
            if model.layers[run.layer].mixer.kv_spec() is not None:
                mem.k_cache, mem.v_cache, mem.space = storage.layer_cache(owner)
            self.memory.append(mem)
        self.windows = [s.window for s in storage.spaces]

    # ---- packing ----------------------------------------------------------------------------
    def prepare(self, entries: Sequence[StepEntry]) -> tuple[StepContext, torch.Tensor, int]:
        """Packs a step into device tensors; returns (context, wanted rows, number of wanted rows).
        Everything a kernel will index with is checked here first."""
        if not entries:
            raise StepError("a step needs at least one entry")
        ps = self.storage.page_size
        vocab, max_pos = self.model.spec.vocab_size, self.model.spec.max_position
        num_spaces = len(self.storage.spaces)
        ids: list[int] = []
        positions: list[int] = []
        seq_of: list[int] = []
        cu = [0]
        starts: list[int] = []
        ctx_lens: list[int] = []
        slots: list[int] = []
        rows: list[int] = []
        tables: list[list[Sequence[int]]] = [[] for _ in range(num_spaces)]
        slot_maps: list[list[int]] = [[] for _ in range(num_spaces)]
        seen: set[int] = set()
        for s, e in enumerate(entries):
            n = len(e.tokens)
            if n == 0:
                raise StepError(f"request {e.seq_id}: an entry feeds at least one token")
            if e.seq_id in seen:
                raise StepError(f"request {e.seq_id} appears twice in one step")
            seen.add(e.seq_id)
            end = e.start + n
            if e.start < 0 or end > max_pos:
                raise StepError(f"request {e.seq_id}: positions {e.start}..{end - 1} exceed the model's {max_pos}")
            lo, hi = min(e.tokens), max(e.tokens)
            if lo < 0 or hi >= vocab:
                raise StepError(f"request {e.seq_id}: token id {lo if lo < 0 else hi} outside the vocabulary of {vocab}")
            for w in e.want:
                if not 0 <= w < n:
                    raise StepError(f"request {e.seq_id}: wanted place {w} is not among its {n} tokens")
                rows.append(cu[-1] + w)
            ids.extend(e.tokens)
            positions.extend(range(e.start, end))
            seq_of.extend([s] * n)
            starts.append(e.start)
            ctx_lens.append(end)
            slots.append(self.view.state_slot(e.seq_id))
            for sp in range(num_spaces):
                table = self.view.block_table(e.seq_id, sp)
                if len(table) * ps < end:
                    raise StepError(f"request {e.seq_id}: {len(table)} pages reserved, positions up to {end - 1} fed")
                first_read = max(0, e.start - self.windows[sp] + 1) if self.windows[sp] else 0
                for j in range(first_read // ps, (end - 1) // ps + 1):
                    if not 0 <= table[j] < self.storage.spaces[sp].num_pages:
                        raise StepError(f"request {e.seq_id}: page {j} of space {sp} is {table[j]}")
                tables[sp].append(table)
                slot_maps[sp].extend(table[p // ps] * ps + p % ps for p in range(e.start, end))
            cu.append(cu[-1] + n)
        T, S, R = len(ids), len(entries), len(rows)
        widths = [max(len(t) for t in tables[sp]) for sp in range(num_spaces)]
        flat: list[int] = ids + positions + seq_of + cu + ctx_lens + slots + rows
        offsets = []
        for sp in range(num_spaces):
            offsets.append(len(flat))
            for t in tables[sp]:
                flat.extend(0 if p == FREED else p for p in t)
                flat.extend([0] * (widths[sp] - len(t)))
        packed = torch.tensor(flat, dtype=torch.int32).to(self.device, non_blocking=True)
        slot_packed = torch.tensor([x for m in slot_maps for x in m], dtype=torch.int64).to(self.device, non_blocking=True)
        o = 0

        def cut(n: int) -> torch.Tensor:
            nonlocal o
            piece = packed[o:o + n]
            o += n
            return piece

        ctx = StepContext(
            num_tokens=T, num_seqs=S, token_ids=cut(T), positions=cut(T), seq_of_token=cut(T), cu_seqlens=cut(S + 1),
            context_lens=cut(S), state_slots=cut(S), slot_mapping=[], block_tables=[],
            host_cu_seqlens=cu, host_starts=starts, host_context_lens=ctx_lens, host_state_slots=slots)
        row_t = cut(R)
        for sp in range(num_spaces):
            ctx.block_tables.append(packed[offsets[sp]:offsets[sp] + S * widths[sp]].view(S, widths[sp]))
            ctx.slot_mapping.append(slot_packed[sp * T:(sp + 1) * T])
        return ctx, row_t, R

    # ---- running ----------------------------------------------------------------------------
    @torch.inference_mode()
    def step(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        """Runs the step; returns float32 logits [wanted, vocab] on the device (an empty tensor
        if nothing is wanted; the tokens' keys and values are written all the same)."""
        ctx, rows, num_rows = self.prepare(entries)
        hidden, residual = self.model.forward(ctx, self.memory)
        if num_rows == 0:
            return torch.empty((0, self.model.spec.vocab_size), dtype=torch.float32, device=self.device)
        return self.model.logits(hidden, residual, rows)

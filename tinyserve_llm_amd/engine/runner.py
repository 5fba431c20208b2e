"""The step function: one batch of (request, its next tokens) through the model, from the cache,
with logits at the wanted places only (tinyserve_llm/engine/model_runner.py:43-133 packs and runs
whole prompt remainders and samples inside; here portions are first-class and logits come out).

A step's entries may be portions of prompts of any length beside single decoded tokens. Each
entry says where its tokens start; the cache manager has already reserved their slots. The step
runs only these tokens, writes their keys and values, attends over the pages, and returns float32
logits [wanted, vocab] in the order of the entries and of their `want` lists.
"""

from __future__ import annotations

import contextlib
import gc
import struct
import sys
import weakref
from array import array
from typing import NamedTuple, Sequence

import torch

from tinyserve_llm_amd.engine.interface import StepMemory, TableView
from tinyserve_llm_amd.models.decoder import DecoderModel
from tinyserve_llm_amd.parts.base import LayerMemory, StepContext


class StepEntry(NamedTuple):          # (a tuple: a step of hundreds of requests makes one for each of them)
    seq_id: int
    tokens: Sequence[int]
    start: int                        # position of tokens[0] in its request
    want: Sequence[int] = ()          # indices into `tokens` whose logits are wanted


class StepError(ValueError):
    pass


class ModelRunner:
    def __init__(self, model: DecoderModel, storage: StepMemory, view: TableView) -> None:
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
        self.graphs: DecodeGraphs | None = None

    # ---- packing ----------------------------------------------------------------------------
    def _pack(self, entries: Sequence[StepEntry], table_widths: list[int] | None = None, pad_to: int = 0):
        """Checks a step on the host and lays it out as flat integer lists. With `table_widths`
        every block table is padded to that width; with `pad_to` the batch is filled up with idle
        one-token rows (position 0, no cache write, page 0) to that many requests."""
        if not entries:
            raise StepError("a step needs at least one entry")
        ps = self.storage.page_size
        vocab, max_pos = self.model.spec.vocab_size, self.model.spec.max_position or sys.maxsize
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
                read = table[first_read // ps:(end - 1) // ps + 1]
                if min(read) < 0 or max(read) >= self.storage.spaces[sp].num_pages:
                    raise StepError(f"request {e.seq_id}: its pages {first_read // ps}..{(end - 1) // ps} of space {sp} "
                                    f"hold {min(read)}..{max(read)}")
                tables[sp].append(table)
                if n == 1:
                    slot_maps[sp].append(table[e.start // ps] * ps + e.start % ps)
                else:
                    p = e.start
                    while p < end:                       # page by page: consecutive positions, consecutive slots
                        page, stop = p // ps, min(end, (p // ps + 1) * ps)
                        base = table[page] * ps - page * ps
                        slot_maps[sp].extend(range(base + p, base + stop))
                        p = stop
            cu.append(cu[-1] + n)
        for s in range(len(entries), pad_to):           # idle rows of a fixed-size batch
            ids.append(0)
            positions.append(0)
            seq_of.append(s)
            starts.append(0)
            ctx_lens.append(1)
            slots.append(0)
            rows.append(cu[-1])
            cu.append(cu[-1] + 1)
            for sp in range(num_spaces):
                tables[sp].append([0])
                slot_maps[sp].append(-1)
        T, S, R = len(ids), len(cu) - 1, len(rows)
        widths = table_widths or [max(len(t) for t in tables[sp]) for sp in range(num_spaces)]
        flat: list[int] = ids + positions + seq_of + cu + ctx_lens + slots + rows
        offsets = []
        for sp in range(num_spaces):
            offsets.append(len(flat))
            for t in tables[sp]:
                if len(t) > widths[sp]:
                    raise StepError(f"a block table of {len(t)} pages exceeds the fixed width {widths[sp]}")
                if self.windows[sp]:
                    flat.extend(p if p >= 0 else 0 for p in t)     # (below 0: pages a window has passed)
                else:
                    flat.extend(t)
                flat.extend([0] * (widths[sp] - len(t)))
        slot_offset = len(flat)
        for m in slot_maps:
            flat.extend(m)
        host = dict(cu=cu, starts=starts, ctx_lens=ctx_lens, slots=slots)
        return flat, (T, S, R, widths, offsets, slot_offset), host

    def _pack_decode(self, entries: Sequence[StepEntry], table_widths: list[int], pad_to: int):
        """`_pack` for steps whose entries all feed one token and want its logits: the same checks
        and the same layout, without the per-token loops."""
        ps = self.storage.page_size
        vocab, max_pos = self.model.spec.vocab_size, self.model.spec.max_position or sys.maxsize
        num_spaces = len(self.storage.spaces)
        S, n = max(pad_to, len(entries)), len(entries)
        ids = [e.tokens[0] for e in entries]
        starts = [e.start for e in entries]
        if len({e.seq_id for e in entries}) != n:
            raise StepError("a request appears twice in one step")
        if n and (min(ids) < 0 or max(ids) >= vocab):
            raise StepError(f"a token id outside the vocabulary of {vocab}")
        if n and (min(starts) < 0 or max(starts) >= max_pos):
            raise StepError(f"a position outside the model's {max_pos}")
        pad = S - n
        slots = [self.view.state_slot(e.seq_id) for e in entries]
        flat = (ids + [0] * pad + starts + [0] * pad + list(range(S)) + list(range(S + 1))
                + [p + 1 for p in starts] + [1] * pad + slots + [0] * pad + list(range(S)))
        offsets, slot_flat = [], []
        for sp in range(num_spaces):
            offsets.append(len(flat))
            width, window, pages = table_widths[sp], self.windows[sp], self.storage.spaces[sp].num_pages
            for e in entries:
                table = self.view.block_table(e.seq_id, sp)
                last = e.start // ps
                if len(table) <= last or len(table) > width:
                    raise StepError(f"request {e.seq_id}: {len(table)} pages reserved for position {e.start} "
                                    f"(fixed width {width})")
                read = table[max(0, e.start - window + 1) // ps if window else 0:last + 1]
                if min(read) < 0 or max(read) >= pages:
                    raise StepError(f"request {e.seq_id}: its pages of space {sp} hold {min(read)}..{max(read)}")
                if window:
                    flat.extend(p if p >= 0 else 0 for p in table)
                else:
                    flat.extend(table)
                flat.extend([0] * (width - len(table)))
                slot_flat.append(table[last] * ps + e.start % ps)
            flat.extend([0] * (pad * width))
            slot_flat.extend([-1] * pad)
        slot_offset = len(flat)
        flat.extend(slot_flat)
        host = dict(cu=list(range(S + 1)), starts=starts + [0] * pad, ctx_lens=[p + 1 for p in starts] + [1] * pad,
                    slots=slots + [0] * pad)
        return flat, (S, S, S, table_widths, offsets, slot_offset), host

    def _context(self, packed: torch.Tensor, dims, host) -> tuple[StepContext, torch.Tensor]:
        T, S, R, widths, offsets, slot_offset = dims
        o = 0

        def cut(n: int) -> torch.Tensor:
            nonlocal o
            piece = packed[o:o + n]
            o += n
            return piece

        ctx = StepContext(
            num_tokens=T, num_seqs=S, token_ids=cut(T), positions=cut(T), seq_of_token=cut(T), cu_seqlens=cut(S + 1),
            context_lens=cut(S), state_slots=cut(S), slot_mapping=[], block_tables=[],
            host_cu_seqlens=host["cu"], host_starts=host["starts"], host_context_lens=host["ctx_lens"],
            host_state_slots=host["slots"], page_size=self.storage.page_size)
        row_t = cut(R)
        for sp in range(len(widths)):
            ctx.block_tables.append(packed[offsets[sp]:offsets[sp] + S * widths[sp]].view(S, widths[sp]))
            ctx.slot_mapping.append(packed[slot_offset + sp * T:slot_offset + (sp + 1) * T])
        return ctx, row_t

    def prepare(self, entries: Sequence[StepEntry]) -> tuple[StepContext, torch.Tensor, int]:
        """Packs a step into device tensors; returns (context, wanted rows, number of wanted rows).
        Everything a kernel will index with is checked here first."""
        flat, dims, host = self._pack(entries)
        # (a list goes into an int32 tensor fastest through the array module)
        packed = torch.frombuffer(array("i", flat), dtype=torch.int32).to(self.device, non_blocking=True)
        ctx, rows = self._context(packed, dims, host)
        return ctx, rows, dims[2]

    # ---- running ----------------------------------------------------------------------------
    @torch.inference_mode()
    def step(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        """Runs the step; returns float32 logits [wanted, vocab] on the device (an empty tensor
        if nothing is wanted; the tokens' keys and values are written all the same)."""
        if self.graphs is not None and self.graphs.takes(entries):
            return self.graphs.run(entries)
        ctx, rows, num_rows = self.prepare(entries)
        hidden, residual = self.model.forward(ctx, self.memory)
        if num_rows == 0:
            return torch.empty((0, self.model.spec.vocab_size), dtype=torch.float32, device=self.device)
        return self.model.logits(hidden, residual, rows)

    @torch.inference_mode()
    def step_sample(self, entries: Sequence[StepEntry], temperatures: Sequence[float], keys: Sequence[int],
                    seed: int) -> torch.Tensor:
        """Runs a step in which every entry wants the logits of exactly one place and draws one token
        from each: int32 [entries], as a device tensor or, from a replayed graph, as `DrawnTokens`
        (`tolist()` gives them either way). `keys[i]` names the draw of entry i (see
        `sampling.sampler`). Decode steps replay a graph that holds the draw as well."""
        if self.graphs is not None and self.graphs.seed == seed and self.graphs.takes(entries):
            return self.graphs.run(entries, (temperatures, keys))
        from tinyserve_llm_amd.sampling.sampler import sample
        return sample(self.step(entries), list(temperatures), list(keys), seed)

    def prepare_decode(self, entries: Sequence[StepEntry], temperatures: Sequence[float], keys: Sequence[int],
                       seed: int, feed: Sequence[int] | None = None):
        """Checks and packs a decode step with its draws ahead of time, on the host alone, while the
        device is busy. The token id of an entry may be a stand-in: `feed[i]` >= 0 then names the row
        of the step before whose drawn token entry i takes (-1: the id given is the real one).
        None if the step is not one the decode graphs take."""
        if self.graphs is not None and self.graphs.seed == seed and self.graphs.takes(entries):
            return self.graphs.prepare(entries, (temperatures, keys), feed)
        return None

    @torch.inference_mode()
    def launch_decode(self, prepared, drawn_before: "DrawnTokens | torch.Tensor | None" = None) -> "DrawnTokens":
        """Starts a step that `prepare_decode` packed; `drawn_before` is what the step before drew
        (`DrawnTokens` or a device tensor, possibly still being computed), from which the entries that
        `feed` named take their ids. Returns the drawn tokens as `DrawnTokens`."""
        return self.graphs.launch(prepared, drawn_before=drawn_before)

    def enable_decode_graphs(self, max_context: int, max_batch: int, seed: int = 0, *, max_graphs: int = 0,
                             memory_budget: int = 0, time_library: bool = True) -> bool:
        """Decode steps (every entry one token whose logits are wanted) are then replayed from HIP
        graphs, one per batch size, instead of being launched kernel by kernel. Only for models
        whose parts all declare `graph_safe`. `seed` is the one the graphs' draws use; `max_graphs`
        and `memory_budget` bound what is kept (0: `DecodeGraphs`' defaults); `time_library` as in
        `DecodeGraphs`. Returns whether graphs are on."""
        if not self.model.graph_safe():
            return False
        self.graphs = DecodeGraphs(self, max_context, max_batch, seed, max_graphs=max_graphs or DecodeGraphs.MAX_GRAPHS,
                                   memory_budget=memory_budget or DecodeGraphs.MEMORY_BUDGET, time_library=time_library)
        return True


class DrawnTokens:
    """The tokens a replayed step drew: on the device, where the graph wrote them (for the step
    started right after it to take its ids from; the graph's next replay overwrites them), and a
    copy on its way to pinned host memory. `tolist()` waits for that copy alone, not for what was
    started on the device after it."""

    def __init__(self, on_device: torch.Tensor, host: torch.Tensor, landed: torch.cuda.Event, n: int,
                 kept: list | None = None) -> None:
        self._on_device, self.host, self.landed, self.n = on_device, host, landed, n
        # the graph these tokens came from and the number of its replay that drew them: the graph's
        # next replay overwrites them on the device, the one after that their landing place on the host
        self._kept, self._replay = kept, kept[8] if kept is not None else 0

    def _replays_since(self) -> int:
        return 0 if self._kept is None else self._kept[8] - self._replay

    @property
    def on_device(self) -> torch.Tensor:
        if self._replays_since() >= 1:
            raise StepError("these tokens are gone from the device: the graph that drew them has been replayed since")
        return self._on_device

    def tolist(self) -> list[int]:
        if self._replays_since() >= 2:
            raise StepError("these tokens are gone: the graph that drew them has been replayed twice since, and its "
                            "two landing places on the host take turns")
        self.landed.synchronize()
        return self.host[:self.n].tolist()


class DecodeGraphs:
    """HIP graphs of the decode step. A graph is captured the first time a (batch size, context
    bucket) pair is met: sizes above 8 round up to a multiple of 8 and idle rows fill the batch;
    the longest context of the batch rounds up to a multiple of 256 positions and fixes the width
    of the block tables, and with it the attention kernels' grids. A graph's inputs live in one
    fixed device buffer that every replay overwrites with one copy from pinned host memory: the
    step's integers, then the draws' keys and temperatures. A graph ends with the logits and with
    the tokens drawn from them; a caller that only wants logits ignores the tokens.

    What is kept is bounded: at most `max_graphs` graphs whose own buffers (the logits above all:
    batch size x vocabulary x 4 bytes each) add up to at most `memory_budget` bytes; beyond either,
    the graph replayed longest ago is dropped (and recorded again if its key comes back). The engine
    sets the budget aside when it sizes the cache pool. `record` makes a graph ahead of its first
    use, so that no request waits for a recording."""

    MAX_GRAPHS = 64
    MEMORY_BUDGET = 2 << 30

    def __init__(self, runner: ModelRunner, max_context: int, max_batch: int, seed: int = 0, *,
                 max_graphs: int = MAX_GRAPHS, memory_budget: int = MEMORY_BUDGET, time_library: bool = True) -> None:
        self.runner = weakref.proxy(runner)     # (the runner owns the graphs: no cycle, so a dropped engine's memory is freed at once)
        self.page_size = runner.storage.page_size
        self.num_spaces = len(runner.storage.spaces)
        self.bucket = max(256, self.page_size)
        self.max_context = max_context
        self.max_batch = max_batch
        self.can_pad = not runner.model.state_plan()
        self.graphs: dict[tuple[int, int], list] = {}      # (batch size, table width) -> kept graph, oldest replay first
        self.max_graphs = max(2, max_graphs)      # (the step before and the step being started may be of two graphs)
        self.memory_budget = memory_budget
        self.recorded = 0                 # graphs recorded so far, dropped ones included
        self.dropped = 0
        # Whether the matrix library's candidates for a batch size are timed when its step is recorded
        # (faster steps; which candidate wins may differ between two runs, and with it the rounding).
        self.time_library = time_library
        self.pool = None
        self.seed = seed                  # of the draws the graphs hold
        from tinyserve_llm_amd.ops import hip
        hip.gemm_library_init()           # its workspace cannot be allocated while a graph is recorded

    def _size(self, n: int) -> int:
        return n if n <= 8 or not self.can_pad else -(-n // 8) * 8

    def takes(self, entries: Sequence[StepEntry]) -> bool:
        if len(entries) > self.max_batch:
            return False
        for e in entries:
            if len(e.tokens) != 1 or len(e.want) != 1 or e.want[0] != 0 or e.start + 1 > self.max_context:
                return False
        return True

    @staticmethod
    def _with_draws(flat: list[int], size: int, draws, feed: Sequence[int] | None = None) -> tuple[torch.Tensor, int]:
        """The upload: `flat`, padded to an even length, then `size` keys (int64, low word first)
        and `size` temperatures (float32) as raw 32-bit words; rows without a draw get key 0 and
        temperature 0. Then `size` rows of the step before that feed the entries (-1: none)."""
        start = len(flat) + (len(flat) & 1)
        words = flat + [0] * (start - len(flat))
        if draws is None:
            words += [0] * (3 * size)
        else:
            temperatures, keys = draws
            n = len(keys)
            for k in keys:                                   # two's complement halves, as int32
                lo, hi = k & 0xFFFFFFFF, (k >> 32) & 0xFFFFFFFF
                words.append(lo - (1 << 32) if lo >= 1 << 31 else lo)
                words.append(hi - (1 << 32) if hi >= 1 << 31 else hi)
            words += [0] * (2 * (size - n))
            words += struct.unpack(f"{n}i", struct.pack(f"{n}f", *temperatures))
            words += [0] * (size - n)
        words += [-1] * size if feed is None else list(feed) + [-1] * (size - len(feed))
        return torch.tensor(words, dtype=torch.int32), start

    def _capture(self, size: int, words: torch.Tensor, start: int, dims, host):
        from tinyserve_llm_amd.ops import hip
        r = self.runner
        host_i32 = torch.empty(len(words), dtype=torch.int32, pin_memory=True)
        dev_i32 = torch.zeros(len(words), dtype=torch.int32, device=r.device)
        host_i32.copy_(words)
        dev_i32.copy_(host_i32, non_blocking=True)
        ctx, rows = r._context(dev_i32, dims, host)
        draw_keys = dev_i32[start:start + 2 * size].view(torch.int64)
        draw_temps = dev_i32[start + 2 * size:start + 3 * size].view(torch.float32)
        # once without capture: libraries set up their workspaces, the kernel library loads, and
        # the matrix library's candidates for this batch size are timed and the fastest kept
        # (this run and the first replay feed the same tokens: keys and values land in the same slots
        # twice, which changes nothing, but a mixer's state would take the step twice, so the state
        # slots are put back as they were. The copies are queued on the current stream before the
        # side stream is told to wait for it: the side stream's run, which writes the slots, then
        # starts after the copies have been taken.)
        states = r.storage.state_tensors()
        before = [t.clone() for t in states]
        side = torch.cuda.Stream(device=r.device)
        side.wait_stream(torch.cuda.current_stream(r.device))
        tuning = hip.library_tuning() if self.time_library else contextlib.nullcontext()
        with tuning, torch.cuda.stream(side):      # (the sweep buffer belongs to the current stream)
            hidden, residual = r.model.forward(ctx, r.memory)
            hip.sample(r.model.logits(hidden, residual, rows), draw_temps, draw_keys, self.seed)
        torch.cuda.current_stream(r.device).wait_stream(side)
        for t, kept in zip(states, before):
            t.copy_(kept)
        torch.cuda.synchronize(r.device)
        graph = torch.cuda.CUDAGraph()

        def body():
            hidden, residual = r.model.forward(ctx, r.memory)
            logits = r.model.logits(hidden, residual, rows)
            return logits, hip.sample(logits, draw_temps, draw_keys, self.seed)

        logits, tokens = self._record(graph, self.pool, body)
        if self.pool is None:
            self.pool = graph.pool()
        # the drawn tokens travel to the host through two pinned buffers in turn: a step may be
        # started before the tokens of the step before it have been read
        landing = [(torch.empty(size, dtype=torch.int32, pin_memory=True), torch.cuda.Event()) for _ in range(2)]
        return [graph, host_i32, dev_i32, logits, tokens, torch.cuda.Event(), landing, 0, 0]    # (.., turn, replays)

    @staticmethod
    def _bytes_of(kept: list) -> int:
        """What a kept graph holds on the device for itself: its inputs, logits and tokens (the
        activations between them lie in the pool that all graphs share)."""
        return sum(t.numel() * t.element_size() for t in (kept[2], kept[3], kept[4]))

    def memory_held(self) -> int:
        return sum(self._bytes_of(k) for k in self.graphs.values())

    def _make_room(self, incoming: int) -> None:
        """Drops the graphs replayed longest ago until one more of `incoming` bytes fits both bounds."""
        while self.graphs and (len(self.graphs) >= self.max_graphs
                               or (len(self.graphs) >= 2 and self.memory_held() + incoming > self.memory_budget)):
            oldest = next(iter(self.graphs))
            # its last replay may still be running, and its tokens on their way to the host
            torch.cuda.current_stream(self.runner.device).synchronize()
            del self.graphs[oldest]
            self.dropped += 1

    def _kept(self, key: tuple[int, int], words: torch.Tensor, start: int, dims, host) -> list:
        """The graph for `key`, recorded now if it is not kept; it becomes the most recently used."""
        kept = self.graphs.pop(key, None)
        if kept is None:
            vocab = self.runner.model.spec.vocab_size
            self._make_room(key[0] * vocab * 4 + 4 * len(words) + 4 * key[0])
            kept = self._capture(key[0], words, start, dims, host)
            self.recorded += 1
        self.graphs[key] = kept
        return kept

    def record(self, batch_size: int, context: int) -> tuple[int, int]:
        """Records the graph that serves `batch_size` requests whose longest context is `context`
        positions, ahead of its first use, from a step of idle rows (position 0, page 0, nothing
        written). Returns the graph's key."""
        if not 1 <= batch_size <= self.max_batch or not 1 <= context <= self.max_context:
            raise StepError(f"no recorded step serves {batch_size} requests of {context} positions "
                            f"(up to {self.max_batch} of {self.max_context})")
        size, width = self._size(batch_size), self._width(context)
        if (size, width) not in self.graphs:
            flat, dims, host = self.runner._pack_decode([], [width] * self.num_spaces, pad_to=size)
            words, start = self._with_draws(flat, size, None)
            self._kept((size, width), words, start, dims, host)
        return size, width

    def _width(self, longest: int) -> int:
        """Pages per block table of the graph that serves contexts up to `longest` positions."""
        reach = min(-(-longest // self.bucket) * self.bucket, -(-self.max_context // self.bucket) * self.bucket)
        return -(-reach // self.page_size)

    @staticmethod
    def _record(graph, pool, body):
        """Runs `body` while the current stream is recorded into `graph`, with garbage collection
        off: an engine that the process has dropped earlier may still be waiting to be collected,
        and destroying its graphs is an operation that a recording forbids (the process then aborts
        in the graph's destructor). What is pending is collected after the recording."""
        collecting = gc.isenabled()
        gc.disable()
        try:
            with torch.cuda.graph(graph, pool=pool):
                return body()
        finally:
            if collecting:
                gc.enable()

    def prepare(self, entries: Sequence[StepEntry], draws=None, feed: Sequence[int] | None = None) -> tuple:
        """The host half of `run`: checks and packs the step. Token ids of entries that `feed`
        names a source row for may be placeholders (any id inside the vocabulary)."""
        if feed is not None and (len(feed) != len(entries) or min(feed) < -1):
            raise StepError("one source row (or -1) per entry")
        size = self._size(len(entries))
        width = self._width(max(e.start + 1 for e in entries))
        flat, dims, host = self.runner._pack_decode(entries, [width] * self.num_spaces, pad_to=size)
        words, start = self._with_draws(flat, size, draws, feed)
        return (size, width), words, start, dims, host, len(entries), draws is not None, feed is not None and max(feed) >= 0

    def launch(self, prepared: tuple, drawn_before: torch.Tensor | None = None) -> torch.Tensor:
        """The device half: uploads the packed step, lets the entries that name a source row take
        their ids from `drawn_before` (the tokens of the step before, on the device) and replays the
        step's graph. Logits [entries, vocab], or the tokens drawn (`DrawnTokens`) if the step was
        prepared with draws."""
        from tinyserve_llm_amd.ops import hip
        key, words, start, dims, host, n, drawn, fed = prepared
        if fed and drawn_before is None:
            raise StepError("the step takes ids from the step before, whose tokens were not given")
        kept = self._kept(key, words, start, dims, host)    # (a recording does not run the step: the replay below does)
        graph, host_i32, dev_i32, logits, tokens, uploaded, landing, turn, _ = kept
        uploaded.synchronize()                  # the last upload from the pinned words has long been made
        host_i32.copy_(words)
        dev_i32.copy_(host_i32, non_blocking=True)
        uploaded.record()
        if fed:
            size = key[0]
            before = drawn_before.on_device if isinstance(drawn_before, DrawnTokens) else drawn_before
            hip.feed_tokens(dev_i32[:n], before.contiguous(), dev_i32[start + 3 * size:start + 3 * size + n])
        graph.replay()
        kept[8] += 1
        if not drawn:
            return logits[:n]
        host_tokens, landed = landing[turn]
        kept[7] = 1 - turn
        # The tokens stay where the graph wrote them. The copy to the host is queued behind this replay
        # and ahead of the next one, and the step after this one takes its ids from here before its own
        # replay is queued (`feed_tokens` above), so the next replay of this graph, which writes the
        # tokens anew, comes after both on the stream.
        host_tokens[:n].copy_(tokens[:n], non_blocking=True)
        landed.record()
        return DrawnTokens(tokens[:n], host_tokens, landed, n, kept)

    def run(self, entries: Sequence[StepEntry], draws=None) -> torch.Tensor:
        """Replays the step's graph. Without `draws` the logits [entries, vocab] come back; with
        `draws` = (temperatures, keys) the tokens drawn from them, int32 [entries]."""
        return self.launch(self.prepare(entries, draws))

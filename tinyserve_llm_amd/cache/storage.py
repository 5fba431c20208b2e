"""Device memory of the cache: key and value pools in pages, grouped by what layers need, and the
slots of fixed-size per-request state (tinyserve_llm/kvcache/storage.py:5-49 has one pool pair
for all layers).

Layers are grouped by the rows they cache (kv heads, head size) and by whether they keep every key
or a window. A group's key pool is laid out [layers of the group, pages, kv_heads, page_size,
head_dim]: layer first, because a step reads one layer's pages at a time and reads them faster
from one compact region (the reference's pool is page first, to copy a page in one piece); within a
page a head's slots lie together, so the attention kernels stream a head's keys from consecutive
memory. The value pool is [layers, pages, kv_heads, head_dim, page_size]: pages hold values
transposed, because the matrix-core product P·V wants, for one dimension, consecutive keys side by
side. All
full-history groups share page space 0: a page id addresses the pools of each of them. Every
window group has a page space of its own.

The pools of bfloat16 caches are cut into pages of 32 slots whatever the page size the manager
counts in (a multiple of 32): page p of the manager is the pool's pages p n .. p n + n - 1, n =
page_size / 32, and slot numbers are the same either way. A 32-key step of the attention kernels
then finds its keys and its values each as one stretch of memory (in a
transposed page of 256 slots a step's values are 64-byte pieces 512 bytes apart: decoding 64
requests over 2,048 keys 54.7 µs a layer, 49.2 with pages of 32). The kernels that read through block
tables are told how many pool pages an entry names; those that write go by slot numbers alone.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from tinyserve_llm_amd.cache.manager import SpaceSpec
from tinyserve_llm_amd.ops import hip
from tinyserve_llm_amd.parts.base import KVSpec


@dataclass
class LayerGroup:
    kv: KVSpec
    space: int
    owners: list[int]                 # run-order indices of the layer runs whose caches live here
    k_pool: torch.Tensor              # [len(owners), pool pages, kv_heads, pool page size, head_dim]
    v_pool: torch.Tensor              # [len(owners), pool pages, kv_heads, head_dim, pool page size]


def plan_spaces(kv_specs: list[KVSpec]) -> tuple[list[tuple[KVSpec, int]], int]:
    """Assigns each distinct KVSpec a page space: window 0 -> space 0, every window size a space of
    its own. Returns ([(spec, space)], number of spaces)."""
    distinct: list[KVSpec] = []
    for kv in kv_specs:
        if kv not in distinct:
            distinct.append(kv)
    windows = sorted({kv.window for kv in distinct if kv.window})
    has_full = any(kv.window == 0 for kv in distinct)
    base = 1 if has_full or not windows else 0
    space_of_window = {w: base + i for i, w in enumerate(windows)}
    return [(kv, 0 if kv.window == 0 else space_of_window[kv.window]) for kv in distinct], max(1, base + len(windows))


def bytes_per_page(cache_plan, page_size: int, dtype: torch.dtype, space: int = 0) -> int:
    """Bytes that one page id of `space` occupies over all layers (keys and values)."""
    assigned, _ = plan_spaces([e.kv for e in cache_plan])
    lookup = dict((kv, s) for kv, s in assigned)
    return sum(2 * page_size * e.kv.num_kv_heads * e.kv.head_dim * dtype.itemsize
               for e in cache_plan if lookup[e.kv] == space)


POOL_PAGE = 32      # slots of a pool's page where the manager's pages are a multiple of it (bfloat16: the matrix-core kernels' step)


class KVStorage:
    def __init__(self, cache_plan, state_plan, num_pages: int | list[int], page_size: int, dtype: torch.dtype,
                 device: torch.device | str, num_state_slots: int) -> None:
        self.page_size = page_size
        # slots of a page of the pools, and the pool pages that make one page of the manager's
        self.pool_page = POOL_PAGE if dtype == torch.bfloat16 and page_size % POOL_PAGE == 0 and \
            (page_size // POOL_PAGE) & (page_size // POOL_PAGE - 1) == 0 else page_size
        self.pages_per_entry = page_size // self.pool_page
        self.dtype = dtype
        self.device = torch.device(device)
        self.num_state_slots = num_state_slots
        assigned, num_spaces = plan_spaces([e.kv for e in cache_plan])
        pages = num_pages if isinstance(num_pages, (list, tuple)) else [num_pages] * num_spaces
        if len(pages) != num_spaces:
            raise ValueError(f"{num_spaces} page spaces but {len(pages)} page counts")
        if any(n * page_size >= 2 ** 31 for n in pages):
            raise ValueError("a page space holds fewer than 2^31 slots (slot numbers travel as int32)")
        windows = [0] * num_spaces
        for kv, s in assigned:
            windows[s] = kv.window
        self.spaces = [SpaceSpec(n, w) for n, w in zip(pages, windows)]
        self.groups: list[LayerGroup] = []
        self._where: dict[int, tuple[int, int]] = {}       # owner run -> (group, layer within group)
        for kv, s in assigned:
            owners = [e.owner for e in cache_plan if e.kv == kv]
            k_shape = (len(owners), pages[s] * self.pages_per_entry, kv.num_kv_heads, self.pool_page, kv.head_dim)
            v_shape = (len(owners), pages[s] * self.pages_per_entry, kv.num_kv_heads, kv.head_dim, self.pool_page)
            group = LayerGroup(kv, s, owners, torch.zeros(k_shape, dtype=dtype, device=self.device),
                               torch.zeros(v_shape, dtype=dtype, device=self.device))
            for j, owner in enumerate(owners):
                self._where[owner] = (len(self.groups), j)
            self.groups.append(group)
        self.states: dict[int, torch.Tensor] = {
            e.run: torch.zeros((num_state_slots, *e.state.shape), dtype=e.state.dtype, device=self.device)
            for e in state_plan}

    @property
    def keeps_state(self) -> bool:
        """Whether some run of the model keeps per-request state (the cache manager then reuses no
        prefix: a skipped token would be missing from the state)."""
        return bool(self.states)

    def layer_cache(self, owner: int) -> tuple[torch.Tensor, torch.Tensor, int]:
        """(k view, v view, page space) of the cache that run `owner` of the order owns; the views
        are addressed [pool pages, pool page size, kv_heads, head_dim] (a permuted view of the pool);
        slot s of the manager's numbering is slot s % pool page size of pool page s // pool page size."""
        g, j = self._where[owner]
        group = self.groups[g]
        return group.k_pool[j].permute(0, 2, 1, 3), group.v_pool[j].permute(0, 3, 1, 2), group.space

    def state(self, run: int) -> torch.Tensor | None:
        return self.states.get(run)

    def state_tensors(self) -> list[torch.Tensor]:
        """Every state tensor, [slots, ...] each (to save and restore around a step that must not count)."""
        return list(self.states.values())

    def copy_slots(self, space: int, src: int, dst: int, num_slots: int) -> None:
        """The first `num_slots` slots of the manager's page `src` into its page `dst`, in every layer."""
        n, size = self.pages_per_entry, self.pool_page
        for group in self.groups:
            if group.space == space:
                for j in range(len(group.owners)):
                    for piece in range(-(-num_slots // size)):
                        slots = min(size, num_slots - piece * size)
                        hip.copy_slots(group.k_pool[j], src * n + piece, dst * n + piece, slots, slot_dim=2)
                        hip.copy_slots(group.v_pool[j], src * n + piece, dst * n + piece, slots, slot_dim=3)

    def copy_state(self, src_slot: int, dst_slot: int) -> None:
        for t in self.states.values():
            t[dst_slot].copy_(t[src_slot])

    def reset_state(self, slot: int) -> None:
        for t in self.states.values():
            t[slot].zero_()

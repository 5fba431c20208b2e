"""Where the engine meets the cache. The step function, the engine loop and trace replay know the
cache only by what stands here: two read-only protocols, the cache's configuration, and one
function that builds device memory and its manager for a model. Everything else of `cache/` is
reached by the scheduler alone, which drives the manager's bookkeeping. The reference draws the
same line in tinyserve_llm/engine/interface.py:34-84 (a view class over its manager and a
`build()`); here the view is a protocol that the manager itself satisfies, and the device memory
has a protocol of its own because the step function hands its tensors to the layers.

A test walks the package's imports and fails if a part, a model or one of these engine modules
reaches into `cache/` another way.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Protocol, Sequence

import torch

from tinyserve_llm_amd.cache.manager import CacheStats, KVCacheManager  # noqa: F401  (CacheStats: part of the step record)
from tinyserve_llm_amd.cache import storage as _storage
from tinyserve_llm_amd.cache.storage import KVStorage


@dataclass(frozen=True)
class CacheConfig:
    block_size: int = 256
    caching: bool = True        # False: no prefix reuse; forks still share pages
    device: str = "cuda"


class TableView(Protocol):
    """Read access to the cache manager's books, valid between reserving a step's slots and committing."""

    def block_table(self, seq_id: int, space: int = 0) -> Sequence[int]:
        """Page ids in token order; an entry below 0 is a page that a window has passed and given back."""

    def state_slot(self, seq_id: int) -> int: ...


class PageSpaceShape(Protocol):
    num_pages: int
    window: int


class StepMemory(Protocol):
    """What the step function needs of the cache's device memory."""

    page_size: int
    spaces: Sequence[PageSpaceShape]
    device: torch.device

    def layer_cache(self, owner: int) -> tuple[torch.Tensor, torch.Tensor, int]:
        """(keys, values, page space) of the cache that run `owner` of the model's order owns, both
        addressed [pages, slots of a page, kv_heads, head_dim]. The views' pages may be shorter than
        `page_size` (a whole number of them to a page, laid out one after the other): slot numbers, which
        count in `page_size`, address the same memory either way, and readers that go through block
        tables learn the ratio from the step's context (`StepContext.page_size`)."""

    def state(self, run: int) -> torch.Tensor | None: ...

    def state_tensors(self) -> list[torch.Tensor]: ...


def bytes_per_page(model, page_size: int, dtype: torch.dtype) -> int:
    """Bytes that one page of the model's main page space takes over all layers, keys and values."""
    return _storage.bytes_per_page(model.cache_plan(), page_size, dtype)


def build_cache(model, num_pages: int | list[int], page_size: int, dtype: torch.dtype, device: torch.device | str,
                num_state_slots: int, caching: bool = True) -> tuple[KVStorage, KVCacheManager]:
    """Device memory for the caches and state slots that `model`'s layers ask for, and the manager
    of its pages. The manager serves as the step function's `TableView`, the storage as its
    `StepMemory`; the scheduler gets the manager itself."""
    storage = KVStorage(model.cache_plan(), model.state_plan(), num_pages, page_size, dtype, device, num_state_slots)
    return storage, KVCacheManager(storage, caching=caching)

"""The cache's device memory: pools cut into pages of 32 slots under a manager that counts in longer
pages, and the copy of a page's leading slots across them."""
import pytest
import torch

from tinyserve_llm_amd.cache.storage import KVStorage, POOL_PAGE
from tinyserve_llm_amd.models.decoder import CachePlanEntry
from tinyserve_llm_amd.parts.base import KVSpec

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype,page,pool_page", [(torch.bfloat16, 256, 32), (torch.bfloat16, 64, 32), (torch.bfloat16, 48, 48),
                                                  (torch.bfloat16, 96, 96), (torch.float32, 256, 256), (torch.bfloat16, 16, 16)])
def test_pools_are_cut_into_pages_of_32_slots_and_slot_numbers_stay(dtype, page, pool_page):
    kv = KVSpec(2, 32, 0)
    storage = KVStorage([CachePlanEntry(0, kv), CachePlanEntry(1, kv)], [], 5, page, dtype, "cuda:0", 4)
    assert storage.pool_page == pool_page and storage.pages_per_entry == page // pool_page
    k, v, space = storage.layer_cache(1)
    assert space == 0 and k.shape == v.shape == (5 * page // pool_page, pool_page, 2, 32)
    assert POOL_PAGE == 32
    # slot s of the manager's numbering: the same element of the flattened views whatever the cut
    slot = 3 * page + page - 1
    k[slot // pool_page, slot % pool_page] = 7.0
    flat_k = k.reshape(-1, 2, 32)                   # (a copy: the view is a permuted one)
    assert float(flat_k[slot].min()) == 7.0 and int((flat_k == 7.0).all(-1).all(-1).sum()) == 1
    # the first slots of page 3 into page 1, in every layer
    for j in range(2):
        kj, vj, _ = storage.layer_cache(j)
        kj.copy_(torch.randn(kj.shape, device="cuda:0").to(dtype))
        vj.copy_(torch.randn(vj.shape, device="cuda:0").to(dtype))
    before = [tuple(t.clone() for t in storage.layer_cache(j)[:2]) for j in range(2)]
    take = page - 5 if page > 8 else 3
    storage.copy_slots(0, 3, 1, take)
    for j in range(2):
        for now, was in zip(storage.layer_cache(j)[:2], before[j]):
            now, was = now.reshape(5, page, 2, 32), was.reshape(5, page, 2, 32)
            assert torch.equal(now[1, :take], was[3, :take]), "the leading slots came over"
            assert torch.equal(now[1, take:], was[1, take:]), "the rest of the page is as it was"
            assert torch.equal(now[[0, 2, 3, 4]], was[[0, 2, 3, 4]]), "no other page was touched"

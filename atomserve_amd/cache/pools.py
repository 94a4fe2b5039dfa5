"""The tensors behind the cache manager's ids.

A paged group has one pool [caches in group, 2 (k, v), num_pages, KV, block_size, D]
in the compute dtype: the block_size keys of one head in one page are contiguous;
the value half of a page is stored transposed, [D, block_size].  It
starts zeroed, so that no slot ever holds a non-finite value
(reference atomserve/kv_cache.py:112-118).  A state group has
[caches in group, max_num_seqs + 1, *shape]: one slot per running request and a last one
(`scrap_slot`) that belongs to nobody, for the rows that only pad a captured step.
"""

import torch

from atomserve_amd.cache.manager import CacheManager


class CachePools:
    def __init__(self, manager: CacheManager, dtype: torch.dtype, device):
        self.manager = manager
        self.dtype = dtype
        self.paged = []
        for g in manager.paged_groups:
            r = g.request
            shape = (len(g.cache_ids), 2, manager.num_blocks, r.num_kv_heads, manager.block_size, r.head_dim)
            self.paged.append(torch.zeros(shape, dtype=dtype, device=device))
        self.state = []
        self.scrap_slot = manager.max_num_seqs
        for g in manager.state_groups:
            shape = (len(g.cache_ids), manager.max_num_seqs + 1, *g.request.shape)
            self.state.append(torch.zeros(shape, dtype=g.request.dtype, device=device))

    def pages(self, cache_id: int):
        """(group index, k_pages, v_pages) of one cache: k_pages [num_pages, KV, block_size, D];
        v_pages [num_pages, KV, D, block_size], each page of values transposed so that the keys
        of one coordinate are contiguous (what the matrix-core kernels read directly)."""
        kind, gi, li = self.manager.group_of_cache[cache_id]
        if kind != "paged":
            raise KeyError(f"cache {cache_id} is not paged")
        k = self.paged[gi][li, 0]
        nb, kv, bs, d = k.shape
        return gi, k, self.paged[gi][li, 1].view(nb, kv, d, bs)

    def state_of(self, cache_id: int):
        """(group index, state tensor [max_num_seqs + 1, *shape]) of one cache."""
        kind, gi, li = self.manager.group_of_cache[cache_id]
        if kind != "state":
            raise KeyError(f"cache {cache_id} holds no fixed-size state")
        return gi, self.state[gi][li]

    @staticmethod
    def bytes_per_block(requests: dict, block_size: int, dtype: torch.dtype) -> int:
        """Memory one page id costs across all paged caches, keys and values
        (reference atomserve/kv_cache.py:129-135)."""
        from atomserve_amd.parts.base import PagedCacheRequest

        item = torch.empty((), dtype=dtype).element_size()
        return sum(2 * r.num_kv_heads * r.head_dim * item * block_size
                   for r in requests.values() if isinstance(r, PagedCacheRequest))  # fmt: skip

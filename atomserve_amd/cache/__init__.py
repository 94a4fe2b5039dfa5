from atomserve_amd.cache.allocator import OutOfPagesError, PageAllocator, blocks_for_tokens, page_hash
from atomserve_amd.cache.manager import CacheManager, RequestCache
from atomserve_amd.cache.pools import CachePools

__all__ = ["CacheManager", "CachePools", "OutOfPagesError", "PageAllocator", "RequestCache",
           "blocks_for_tokens", "page_hash"]  # fmt: skip

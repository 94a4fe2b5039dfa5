"""The cache manager: which pages and state slots each request holds, in every group.

Mixers ask for caches (`parts.base.PagedCacheRequest`, `StateCacheRequest`).  Caches
with the same needs form a group:

  paged group   keys and values in pages; one pool, one `PageAllocator` and one block
                table per request for all caches of the group.  A group with a window
                gives back the pages that every future query has left behind.
  state group   a fixed-size state per running request: one slot id per request,
                valid in every state group.

Everything here is bookkeeping over integers (no tensors): the scheduler decides with
it who gets memory, without touching the GPU.  `cache.pools.CachePools` holds the
tensors that the ids index.
"""

from dataclasses import dataclass, field

from atomserve_amd.cache.allocator import PageAllocator, blocks_for_tokens, page_hash
from atomserve_amd.parts.base import PagedCacheRequest, StateCacheRequest

RELEASED = -1  # block-table entry of a page that a window has passed and given back


@dataclass
class PagedGroup:
    index: int
    request: PagedCacheRequest
    cache_ids: list
    allocator: PageAllocator

    @property
    def window(self) -> int:
        return self.request.window


@dataclass
class StateGroup:
    index: int
    request: StateCacheRequest
    cache_ids: list


@dataclass
class RequestCache:
    """What one request holds: a block table per paged group and, if the model keeps
    fixed-size state, one slot."""

    tables: list  # [group] -> list of page ids, position // block_size -> page (or RELEASED)
    hashes: list = field(default_factory=list)  # prefix hash of each full, computed page
    state_slot: int = -1


class CacheManager:
    def __init__(self, requests: dict, block_size: int, num_blocks: int, max_num_seqs: int):
        """requests: cache id -> PagedCacheRequest | StateCacheRequest (from the model)."""
        self.block_size = block_size
        self.num_blocks = num_blocks
        self.max_num_seqs = max_num_seqs
        self.paged_groups: list = []
        self.state_groups: list = []
        self.group_of_cache: dict = {}  # cache id -> ("paged" | "state", group index, index in group)
        for cid in sorted(requests):
            req = requests[cid]
            if isinstance(req, PagedCacheRequest):
                groups, kind = self.paged_groups, "paged"
            elif isinstance(req, StateCacheRequest):
                groups, kind = self.state_groups, "state"
            else:
                raise TypeError(f"cache {cid}: unknown request {req!r}")
            for g in groups:
                if g.request == req:
                    break
            else:
                if kind == "paged":
                    g = PagedGroup(len(groups), req, [], PageAllocator(num_blocks))
                else:
                    g = StateGroup(len(groups), req, [])
                groups.append(g)
            self.group_of_cache[cid] = (kind, g.index, len(g.cache_ids))
            g.cache_ids.append(cid)
        self._free_slots = list(range(max_num_seqs - 1, -1, -1)) if self.state_groups else []
        # A prefix can be reused only where the cached content is a function of the token
        # prefix at page granularity: all keys kept, and no state outside the pages.
        self.prefix_reuse_possible = (
            bool(self.paged_groups) and not self.state_groups and all(g.window == 0 for g in self.paged_groups)
        )

    # ---- counts -----------------------------------------------------------------------
    @property
    def num_free(self) -> int:
        """Free pages of the scarcest group."""
        return min((g.allocator.num_free for g in self.paged_groups), default=self.num_blocks)

    @property
    def num_cached(self) -> int:
        return max((g.allocator.num_cached for g in self.paged_groups), default=0)

    @property
    def num_free_slots(self) -> int:
        return len(self._free_slots)

    def new_request(self) -> RequestCache:
        return RequestCache(tables=[[] for _ in self.paged_groups])

    # ---- pages ------------------------------------------------------------------------
    def reserve(self, rc: RequestCache, num_computed: int, num_new: int) -> bool:
        """Grow every table to hold positions < num_computed + num_new, and take a state slot
        if the model needs one.  All or nothing: on False nothing was taken."""
        need = blocks_for_tokens(num_computed + num_new, self.block_size)
        missing = [need - len(t) for t in rc.tables]
        for g, m in zip(self.paged_groups, missing):
            if m > g.allocator.num_free:
                return False
        if self.state_groups and rc.state_slot < 0 and not self._free_slots:
            return False
        for g, m, table in zip(self.paged_groups, missing, rc.tables):
            if m > 0:
                table.extend(g.allocator.allocate(m))
        if self.state_groups and rc.state_slot < 0:
            rc.state_slot = self._free_slots.pop()
        return True

    def reserve_all(self, wanted) -> bool:
        """`reserve` for several requests of one step together: wanted = [(rc, num_computed, num_new)],
        each request at most once.  All or nothing: on False no request has taken anything."""
        short = [0] * len(self.paged_groups)
        slots = 0
        for rc, num_computed, num_new in wanted:
            need = blocks_for_tokens(num_computed + num_new, self.block_size)
            for g, table in enumerate(rc.tables):
                short[g] += max(0, need - len(table))
            slots += 1 if self.state_groups and rc.state_slot < 0 else 0
        if any(m > g.allocator.num_free for g, m in zip(self.paged_groups, short)) or slots > len(self._free_slots):
            return False
        for rc, num_computed, num_new in wanted:
            if not self.reserve(rc, num_computed, num_new):
                raise RuntimeError("pages counted as free could not be taken")
        return True

    def release_behind_window(self, rc: RequestCache, num_computed: int) -> int:
        """Give back the pages of windowed groups that no query at a position >= num_computed
        can see any more.  Returns how many pages were freed."""
        freed = 0
        for g, table in zip(self.paged_groups, rc.tables):
            if g.window <= 0:
                continue
            first_visible = num_computed - g.window + 1  # the oldest key the next query sees
            dead = min(len(table), max(0, first_visible) // self.block_size)
            pages = [table[b] for b in range(dead) if table[b] != RELEASED]
            if pages:
                g.allocator.free(pages)
                for b in range(dead):
                    table[b] = RELEASED
                freed += len(pages)
        return freed

    def release(self, rc: RequestCache) -> None:
        """Give back everything the request holds (finish, abort or preemption)."""
        for g, table in zip(self.paged_groups, rc.tables):
            g.allocator.free([p for p in table if p != RELEASED])
        # new lists, not cleared ones: whoever still holds the old tables (a step packed earlier)
        # can tell that they no longer describe this request
        rc.tables = [[] for _ in self.paged_groups]
        rc.hashes.clear()
        if rc.state_slot >= 0:
            self._free_slots.append(rc.state_slot)
            rc.state_slot = -1

    # ---- prefix reuse (reference atomserve/scheduler.py:214-250) ------------------------
    def adopt_cached_prefix(self, rc: RequestCache, token_ids: list) -> int:
        """Point the request's empty tables at pages that already hold its leading full pages;
        stops at the first page missing in any group, and always leaves at least one token to
        compute.  Returns the number of tokens covered."""
        if not self.prefix_reuse_possible or any(rc.tables):
            return 0
        bs, parent = self.block_size, b""
        for i in range((len(token_ids) - 1) // bs):
            h = page_hash(parent, token_ids[i * bs : (i + 1) * bs])
            pages = [g.allocator.lookup(h) for g in self.paged_groups]
            if any(p is None for p in pages):
                break
            for g, p, table in zip(self.paged_groups, pages, rc.tables):
                g.allocator.acquire(p)
                table.append(p)
            rc.hashes.append(h)
            parent = h
        return len(rc.hashes) * bs

    def publish_full_pages(self, rc: RequestCache, token_ids: list, num_computed: int) -> None:
        """Name every page that is now full of computed tokens, so later requests can reuse it."""
        if not self.prefix_reuse_possible:
            return
        bs = self.block_size
        while len(rc.hashes) < num_computed // bs:
            i = len(rc.hashes)
            h = page_hash(rc.hashes[-1] if i else b"", token_ids[i * bs : (i + 1) * bs])
            for g, table in zip(self.paged_groups, rc.tables):
                g.allocator.register(table[i], h)
            rc.hashes.append(h)

    def check(self) -> None:
        for g in self.paged_groups:
            g.allocator.check()

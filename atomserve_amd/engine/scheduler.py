"""The scheduler: every step, which requests run and how many tokens each
(policy of reference atomserve/scheduler.py:88-269, without speculative look-ahead).

Continuous batching under two limits, `max_num_seqs` running requests and
`max_num_batched_tokens` tokens per step:

  1. Running requests first, oldest first: one token for a decode, or the next portion
     of a prompt.  If the cache has no room for one, the most recently admitted request
     is preempted: everything it holds is given back, it returns to the front of the
     queue and is recomputed from its tokens later.  A request never evicts one that
     was already scheduled in the same step.
  2. Waiting requests are admitted first come, first served, while budget, request limit
     and free pages allow; never in a step that had to preempt.

A prompt takes whatever budget is left and continues in the next step (chunked
prefill).  On admission a request first adopts cached pages of its prefix; after each
step its newly full pages are published, and pages behind a window are given back.

Bookkeeping only (sequences, page ids): no tensors, testable without a GPU.
"""

from collections import deque
from dataclasses import dataclass, field

from atomserve_amd.cache.manager import CacheManager
from atomserve_amd.config.engine_config import EngineConfig
from atomserve_amd.engine.sequence import Sequence, SequenceStatus


@dataclass
class SchedulerOutput:
    """The plan of one step: seqs[i] runs its next num_new_tokens[i] tokens; `preempted` were
    evicted to make room and are waiting again."""

    seqs: list = field(default_factory=list)
    num_new_tokens: list = field(default_factory=list)
    preempted: list = field(default_factory=list)

    @property
    def num_tokens(self) -> int:
        return sum(self.num_new_tokens)


class Scheduler:
    def __init__(self, config: EngineConfig, eos_token_ids=frozenset(), manager: CacheManager = None):
        """manager: the model's cache manager; without one, a single group of full attention
        pages is assumed (enough for scheduling decisions on their own)."""
        self.config = config
        self.eos_token_ids = frozenset(eos_token_ids)
        if manager is None:
            from atomserve_amd.parts.base import PagedCacheRequest

            manager = CacheManager({0: PagedCacheRequest(1, 1)}, config.block_size, config.num_blocks,
                                   config.max_num_seqs)  # fmt: skip
        if manager.block_size != config.block_size or manager.num_blocks != config.num_blocks:
            raise ValueError("cache manager and engine configuration disagree on the pool")
        self.manager = manager
        self.waiting: deque = deque()
        self.running: list = []  # in admission order

    @property
    def allocator(self):
        """The first paged group's allocator (the only one for a model with one kind of cache)."""
        return self.manager.paged_groups[0].allocator

    def add(self, seq: Sequence) -> None:
        seq.cache = self.manager.new_request()
        self.waiting.append(seq)

    @property
    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    # ---- planning ---------------------------------------------------------------------
    def schedule(self) -> SchedulerOutput:
        budget = self.config.max_num_batched_tokens
        out = SchedulerOutput()

        for seq in list(self.running):
            if seq.status is not SequenceStatus.RUNNING:
                continue  # preempted earlier in this loop
            n = min(seq.num_tokens - seq.num_computed_tokens, budget)
            if n == 0:
                continue  # budget spent: it waits for the next step
            while not self.manager.reserve(seq.cache, seq.num_computed_tokens, n):
                victim = self.running[-1]  # the newest has the least work to redo
                self._preempt(victim)
                out.preempted.append(victim)
                if victim is seq:
                    break
            if seq.status is SequenceStatus.RUNNING:
                out.seqs.append(seq)
                out.num_new_tokens.append(n)
                budget -= n

        while self.waiting and not out.preempted and len(self.running) < self.config.max_num_seqs:
            seq = self.waiting[0]
            if self.config.enable_prefix_caching:
                self._adopt_prefix(seq)
            n = min(seq.num_tokens - seq.num_computed_tokens, budget)
            if n == 0 or not self.manager.reserve(seq.cache, seq.num_computed_tokens, n):
                self.manager.release(seq.cache)  # undo a prefix hit; retry next step
                seq.num_computed_tokens = seq.num_cached_tokens = 0
                break
            self.waiting.popleft()
            seq.status = SequenceStatus.RUNNING
            self.running.append(seq)
            out.seqs.append(seq)
            out.num_new_tokens.append(n)
            budget -= n
        return out

    # ---- after the step ---------------------------------------------------------------
    def update(self, out: SchedulerOutput, results) -> list:
        """Append new tokens, retire finished requests, advance the rest.  Returns
        (sequence, its new tokens) for every sequence that got any."""
        new_tokens = []
        for seq, result in zip(out.seqs, results, strict=True):
            if seq.status is not SequenceStatus.RUNNING:
                continue  # finished or aborted while the step was on its way: its result is dropped
            appended = []
            for token in result.tokens:
                seq.token_ids.append(token)
                appended.append(token)
                reason = self._finish_reason(seq, token)
                if reason:
                    self._finish(seq, reason)
                    break
            if appended:
                new_tokens.append((seq, appended))
            if seq.status is SequenceStatus.FINISHED:
                continue
            # The newest token is never computed yet: its keys come with the next step.
            seq.num_computed_tokens = min(result.num_computed, seq.num_tokens - 1)
            if self.config.enable_prefix_caching:
                self.manager.publish_full_pages(seq.cache, seq.token_ids, seq.num_computed_tokens)
            self.manager.release_behind_window(seq.cache, seq.num_computed_tokens)
        return new_tokens

    def abort(self, seq_id: int):
        for seq in [*self.waiting, *self.running]:
            if seq.id == seq_id:
                if seq in self.waiting:
                    self.waiting.remove(seq)
                self._finish(seq, "abort")
                return seq
        return None

    # ---- internals --------------------------------------------------------------------
    def _finish_reason(self, seq: Sequence, token: int):
        if token in self.eos_token_ids and not seq.params.ignore_eos:
            return "stop"
        if seq.num_output_tokens >= seq.params.max_tokens:
            return "length"
        if seq.num_tokens >= self.config.max_model_len:
            return "length"
        return None

    def _adopt_prefix(self, seq: Sequence) -> None:
        covered = self.manager.adopt_cached_prefix(seq.cache, seq.token_ids)
        seq.num_computed_tokens = covered
        if not seq.num_output_tokens:  # count hits on the prompt, not on recomputing a preempted reply
            seq.num_cached_tokens = covered

    def _preempt(self, seq: Sequence) -> None:
        self.running.remove(seq)
        self.manager.release(seq.cache)
        seq.num_computed_tokens = 0
        seq.status = SequenceStatus.WAITING
        self.waiting.appendleft(seq)

    def _finish(self, seq: Sequence, reason: str) -> None:
        if seq in self.running:
            self.running.remove(seq)
        self.manager.release(seq.cache)
        seq.status = SequenceStatus.FINISHED
        seq.finish_reason = reason

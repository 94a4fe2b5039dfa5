"""The scheduler: for every step, which requests run and how many tokens each brings.

The policy is the reference's (atomserve/scheduler.py:88-269, without its speculative
look-ahead): continuous batching under two limits, `max_num_seqs` requests holding cache
and `max_num_batched_tokens` tokens a step.

  * Requests that already run come first, in the order they were admitted: one token for
    a request that decodes, the next portion of its prompt for one that is still reading.
  * A prompt takes what is left of the step's token budget and goes on in the next step
    (chunked prefill); a request the budget does not reach sits the step out.
  * When the cache has no page for a request, the request admitted last gives back all it
    holds and returns to the head of the queue, to be recomputed from its tokens later.
    Eviction always starts at the newest, so nothing planned earlier in the same step (all
    older) is ever taken away again.
  * New requests are admitted first come, first served, while places, budget and pages
    allow, and never in a step that had to evict.  An admitted request first adopts cached
    pages of its prefix; after every step its newly filled pages are published and pages
    behind a window go back to the pool.

A step is described by a `StepPlan`.  Steps form a pipeline: while the running requests
do nothing but decode, `plan_ahead` describes the step after one that is still on the GPU,
so the engine can launch it before it has read the first one's tokens.

Bookkeeping only (sequences and page ids, no tensors): it runs without a GPU.
"""

from collections import deque
from dataclasses import dataclass, field

from atomserve_amd.cache.manager import CacheManager
from atomserve_amd.config.engine_config import EngineConfig
from atomserve_amd.engine.sequence import Sequence, SequenceStatus


@dataclass
class StepPlan:
    """One step: seqs[i] brings its next num_new_tokens[i] tokens.  `preempted` lost their cache
    to make room and wait again.  `ahead`: planned while the step before was still unread, so
    every request brings the one token that step will give it."""

    seqs: list = field(default_factory=list)
    num_new_tokens: list = field(default_factory=list)
    preempted: list = field(default_factory=list)
    ahead: bool = False

    def give(self, seq: Sequence, count: int) -> None:
        self.seqs.append(seq)
        self.num_new_tokens.append(count)

    @property
    def num_tokens(self) -> int:
        return sum(self.num_new_tokens)


SchedulerOutput = StepPlan  # the reference's name for it (atomserve/scheduler.py:48-66)


class Scheduler:
    def __init__(self, config: EngineConfig, eos_token_ids=frozenset(), manager: CacheManager = None):
        """manager: the model's cache manager.  Without one, a single group of pages that keeps
        every key stands in, which is all that scheduling decisions need."""
        if manager is None:
            from atomserve_amd.parts.base import PagedCacheRequest

            manager = CacheManager({0: PagedCacheRequest(1, 1)}, config.block_size, config.num_blocks,
                                   config.max_num_seqs)  # fmt: skip
        if (manager.block_size, manager.num_blocks) != (config.block_size, config.num_blocks):
            raise ValueError("cache manager and engine configuration disagree on the pool")
        self.config = config
        self.manager = manager
        self.eos_token_ids = frozenset(eos_token_ids)
        self.waiting: deque = deque()  # head first
        self.running: list = []  # oldest admission first

    # ---- what the engine asks -----------------------------------------------------------
    @property
    def has_work(self) -> bool:
        return bool(self.running) or bool(self.waiting)

    def add(self, seq: Sequence) -> None:
        seq.cache = self.manager.new_request()
        self.waiting.append(seq)

    def abort(self, seq_id: int):
        """Ends the request wherever it is; returns it, or None if it is not known (any more)."""
        for place in (self.running, self.waiting):
            for seq in place:
                if seq.id == seq_id:
                    place.remove(seq)
                    self._retire(seq, "abort")
                    return seq
        return None

    # ---- planning -----------------------------------------------------------------------
    def schedule(self) -> StepPlan:
        plan = StepPlan()
        left = self.config.max_num_batched_tokens
        # The requests that run already.  Evictions shorten the list from its end only, so walking
        # it by index meets every survivor once and stops when the walk itself was evicted.
        at = 0
        while at < len(self.running):
            seq = self.running[at]
            at += 1
            share = min(seq.num_tokens - seq.num_computed_tokens, left)
            if share > 0 and self._make_room(seq, share, plan):
                plan.give(seq, share)
                left -= share
        if plan.preempted:
            return plan  # whoever was evicted is first in line; nobody new overtakes it
        while self.waiting and left > 0 and len(self.running) < self.config.max_num_seqs:
            seq = self.waiting[0]
            covered = self.manager.adopt_cached_prefix(seq.cache, seq.token_ids) if self.config.enable_prefix_caching else 0
            share = min(seq.num_tokens - covered, left)
            if not self.manager.reserve(seq.cache, covered, share):
                self.manager.release(seq.cache)  # the adopted pages too: it is looked up again next time
                break  # strictly in order: nobody behind it is tried
            self.waiting.popleft()
            self.running.append(seq)
            seq.status = SequenceStatus.RUNNING
            seq.num_computed_tokens = covered
            if seq.num_output_tokens == 0:  # a hit while recomputing an evicted reply is no hit on the prompt
                seq.num_cached_tokens = covered
            plan.give(seq, share)
            left -= share
        return plan

    def plan_ahead(self, previous: StepPlan):
        """The decode step that follows `previous` while `previous` is still unread, or None if that
        step is not certain yet.  It is certain when `previous` gives every running request exactly
        one new token, none of them can end by length with it, nobody waits for a place that is free,
        and every request has a page for one more position (taken here, all or none: making room is
        `schedule`'s decision).  A request that `previous` ends on an end-of-sequence token still takes
        part; its result is dropped when the step is read."""
        if previous.preempted or len(previous.seqs) != len(self.running):
            return None
        if self.waiting and len(self.running) < self.config.max_num_seqs:
            return None  # schedule() may admit somebody; with every place taken the queue cannot move
        longest = self.config.max_model_len
        for seq, mine, count in zip(self.running, previous.seqs, previous.num_new_tokens):
            if seq is not mine or seq.status is not SequenceStatus.RUNNING or not seq.reaches_end(count):
                return None
            if seq.num_output_tokens + 1 >= seq.params.max_tokens or seq.num_tokens + 1 >= longest:
                return None  # the coming token is its last
        if not self.manager.reserve_all([(seq.cache, seq.num_tokens, 1) for seq in self.running]):
            return None
        return StepPlan(seqs=list(self.running), num_new_tokens=[1] * len(self.running), ahead=True)

    # ---- after a step -------------------------------------------------------------------
    def update(self, plan: StepPlan, results) -> list:
        """Takes a step's results in: new tokens are appended until one ends its request, the others
        move on.  Returns [(sequence, the tokens it gained)]."""
        gained = []
        for seq, result in zip(plan.seqs, results, strict=True):
            if seq.status is not SequenceStatus.RUNNING:
                continue  # ended or evicted while the step was on its way: nothing of it is kept
            kept = self._append(seq, result.tokens)
            if kept:
                gained.append((seq, kept))
            if seq.status is SequenceStatus.RUNNING:
                self._move_on(seq, result.num_computed)
        return gained

    # ---- pieces -------------------------------------------------------------------------
    def _make_room(self, seq: Sequence, count: int, plan: StepPlan) -> bool:
        """Pages for `count` more tokens of a running request, evicting from the newest request down
        until they are there.  False if `seq` itself had to go."""
        while not self.manager.reserve(seq.cache, seq.num_computed_tokens, count):
            loser = self.running.pop()
            self.manager.release(loser.cache)
            loser.num_computed_tokens = 0
            loser.status = SequenceStatus.WAITING
            self.waiting.appendleft(loser)
            plan.preempted.append(loser)
            if loser is seq:
                return False
        return True

    def _append(self, seq: Sequence, tokens) -> list:
        kept = []
        for token in tokens:
            seq.token_ids.append(token)
            kept.append(token)
            reason = self._ends_with(seq, token)
            if reason is not None:
                self.running.remove(seq)
                self._retire(seq, reason)
                break
        return kept

    def _ends_with(self, seq: Sequence, token: int):
        """Why the token just appended is the request's last, or None.  An end-of-sequence token is
        part of the reply (reference atomserve/scheduler.py:177-185)."""
        if not seq.params.ignore_eos and token in self.eos_token_ids:
            return "stop"
        if seq.num_output_tokens >= seq.params.max_tokens or seq.num_tokens >= self.config.max_model_len:
            return "length"
        return None

    def _move_on(self, seq: Sequence, num_computed: int) -> None:
        # the newest token has no key yet: it comes with the next step
        seq.num_computed_tokens = min(num_computed, seq.num_tokens - 1)
        if self.config.enable_prefix_caching:
            self.manager.publish_full_pages(seq.cache, seq.token_ids, seq.num_computed_tokens)
        self.manager.release_behind_window(seq.cache, seq.num_computed_tokens)

    def _retire(self, seq: Sequence, reason: str) -> None:
        self.manager.release(seq.cache)
        seq.status = SequenceStatus.FINISHED
        seq.finish_reason = reason

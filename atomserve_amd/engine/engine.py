"""The engine: one loop that owns the GPU (reference atomserve/engine.py:1-264).

    take new requests and aborts from the inbox -> scheduler
    plan    = scheduler.schedule()
    results = runner.execute(plan)        one pass over the GPU and one sampling call
    scheduler.update(plan, results)
    push each new token to its request's handle

While nothing changes among the running requests (all decode, nobody waits, nobody reaches its
length), the next decode step goes to the GPU before this one's tokens are read: the GPU passes
the sampled tokens on by itself, and the host's share of a step is hidden behind the GPU's.

Clients on any thread talk to it through queues only: one inbox for submit and abort,
one outbox per request that streams its tokens back.  It deals in token ids only.
"""

import itertools
import queue
import random
import sys
import threading
import time
import traceback
from dataclasses import dataclass
from typing import Optional

from atomserve_amd.cache.manager import CacheManager
from atomserve_amd.config.engine_config import EngineConfig
from atomserve_amd.engine.runner import ModelRunner
from atomserve_amd.engine.scheduler import Scheduler, SchedulerOutput
from atomserve_amd.engine.sequence import SamplingParams, Sequence, SequenceStatus
from atomserve_amd.kernels import ops


@dataclass
class _Finished:
    reason: str  # "stop", "length", "abort" or "error"
    error: Optional[BaseException] = None


class RequestHandle:
    """The client's end of one request: iterate it to receive token ids as they are made;
    afterwards `finish_reason` and the timing fields are set."""

    def __init__(self, request_id: int, engine: "Engine", num_prompt_tokens: int):
        self.id = request_id
        self.num_prompt_tokens = num_prompt_tokens
        self.num_output_tokens = 0
        self.num_cached_tokens = 0
        self.finish_reason: Optional[str] = None
        self.submitted_at = time.perf_counter()
        self.first_token_at: Optional[float] = None
        self.finished_at: Optional[float] = None
        self._engine = engine
        self._outbox: queue.SimpleQueue = queue.SimpleQueue()

    def __iter__(self):
        while True:
            event = self._outbox.get()
            if isinstance(event, _Finished):
                self.finish_reason = event.reason
                if event.error is not None:
                    raise RuntimeError("engine step failed") from event.error
                return
            yield event

    def abort(self) -> None:
        self._engine.abort(self.id)

    @property
    def ttft(self):
        """Seconds from submit to the first token."""
        return None if self.first_token_at is None else self.first_token_at - self.submitted_at

    @property
    def decode_tokens_per_s(self):
        if self.first_token_at is None or self.finished_at is None or self.num_output_tokens < 2:
            return None
        return (self.num_output_tokens - 1) / max(self.finished_at - self.first_token_at, 1e-9)


class Engine:
    def __init__(self, runner, scheduler: Scheduler, seed: Optional[int] = None):
        self.runner = runner
        self.scheduler = scheduler
        self._inbox: queue.SimpleQueue = queue.SimpleQueue()
        self._handles: dict = {}
        self._ids = itertools.count()
        self._thread: Optional[threading.Thread] = None
        self._stopping = False
        self._rng = random.Random(seed)  # seeds of the requests that bring none
        self._in_flight = None  # (plan, pending step) of a decode step sent to the GPU ahead of its turn
        self.run_ahead = True
        self.num_steps = 0
        self.last_batch_seqs = 0
        self.last_batch_tokens = 0
        self.num_prompt_tokens = 0
        self.num_cached_prompt_tokens = 0
        self.num_generated_tokens = 0
        self.num_preemptions = 0

    # ---- client side (any thread) ---------------------------------------------------
    def submit(self, prompt_ids, params: SamplingParams) -> RequestHandle:
        limit = self.scheduler.config.max_model_len
        if not 0 < len(prompt_ids) < limit:
            raise ValueError(f"prompt has {len(prompt_ids)} tokens; must be 1 to {limit - 1}")
        if params.max_tokens < 1:
            raise ValueError("max_tokens must be at least 1")
        vocab = getattr(self.runner, "vocab_size", None)
        if vocab is not None and any(not 0 <= int(t) < vocab for t in prompt_ids):
            raise ValueError(f"prompt holds a token id outside the vocabulary of {vocab}")
        request_id = next(self._ids)
        handle = RequestHandle(request_id, self, len(prompt_ids))
        seq = Sequence(request_id, [int(t) for t in prompt_ids], params)
        if params.seed is None:
            seq.noise_seed = self._rng.getrandbits(63)
        self._inbox.put(("add", seq, handle))
        return handle

    def abort(self, request_id: int) -> None:
        self._inbox.put(("abort", request_id))

    def start(self) -> None:
        self._thread = threading.Thread(target=self._loop, name="atomserve-engine", daemon=True)
        self._thread.start()

    def shutdown(self) -> None:
        self._stopping = True
        self._inbox.put(("wake",))
        if self._thread is not None:
            self._thread.join()

    def generate(self, prompts, params: SamplingParams) -> list:
        """Run prompts to completion on the calling thread; all are submitted first, so they
        are batched together (reference atomserve/engine.py:137-146)."""
        handles = [self.submit(p, params) for p in prompts]
        while self.step():
            pass
        return [list(h) for h in handles]

    def warm_up(self) -> int:
        """Before serving: the decode steps of every batch size up to max_num_seqs are captured now
        (kernels are compiled and loaded, the library's candidates tried) rather than at their
        first use.  Returns the number of graphs captured; 0 where decode steps run uncaptured."""
        graphs = getattr(self.runner, "decode_graphs", None)
        if graphs is None:
            return 0
        return graphs.capture_ahead(self.scheduler.config.max_num_seqs)

    def stats(self) -> dict:
        s = self.scheduler
        total = s.manager.num_blocks
        used = total - s.manager.num_free
        return {
            "running": len(s.running),
            "waiting": len(s.waiting),
            "kv_blocks_used": used,
            "kv_blocks_total": total,
            "kv_usage": used / total,
            "kv_blocks_cached": s.manager.num_cached,
            "steps": self.num_steps,
            "last_batch_seqs": self.last_batch_seqs,
            "last_batch_tokens": self.last_batch_tokens,
            "prompt_tokens": self.num_prompt_tokens,
            "cached_prompt_tokens": self.num_cached_prompt_tokens,
            "generated_tokens": self.num_generated_tokens,
            "preemptions": self.num_preemptions,
        }

    # ---- engine side (one thread) ---------------------------------------------------
    def step(self) -> bool:
        """One scheduling step; False when there is nothing to do."""
        self._drain_inbox(block=False)
        flight, self._in_flight = self._in_flight, None
        if flight is not None:
            out, pending = flight  # planned and sent to the GPU during the step before
        else:
            if not self.scheduler.has_work:
                return False
            out = self.scheduler.schedule()
            if not out.seqs:
                raise RuntimeError("scheduler has work but scheduled nothing")
            launch = getattr(self.runner, "launch", None)
            pending = launch(out) if launch is not None else None
        sent = None
        if pending is None:
            results = self.runner.execute(out)
        else:
            ahead = self._plan_ahead(out)
            if ahead is not None:
                sent = (ahead, self.runner.launch(ahead, after=pending))
            results = pending.results()
        new_tokens = self.scheduler.update(out, results)
        self._in_flight = sent  # only now: a step that failed on the way leaves nothing behind

        now = time.perf_counter()
        self.num_steps += 1
        self.num_preemptions += len(out.preempted)
        self.last_batch_seqs, self.last_batch_tokens = len(out.seqs), out.num_tokens
        for seq, tokens in new_tokens:
            handle = self._handles[seq.id]
            if handle.first_token_at is None:
                handle.first_token_at = now
            handle.num_output_tokens += len(tokens)
            self.num_generated_tokens += len(tokens)
            for token in tokens:
                handle._outbox.put(token)
            if seq.status is SequenceStatus.FINISHED:
                self._close(seq)
        return True

    def _plan_ahead(self, out):
        """The decode step after `out`, if it is certain but for its tokens: `out` gives every running
        request a token, nobody can be admitted or has left, nobody reaches its length with that token, no sampling
        setting needs the tokens on the host, and every request has a page for one more position.  A
        request that ends on an end-of-sequence token in `out` still takes part in the step ahead; its
        result there is dropped and its pages, given back at once, may be written once more, which is
        harmless: whoever gets them next writes after that, in the order of the GPU's queue."""
        s = self.scheduler
        can = getattr(self.runner, "can_run_ahead", None)
        if not self.run_ahead or can is None or out.preempted or not self._inbox.empty():
            return None
        if s.waiting and len(s.running) < s.config.max_num_seqs:
            return None  # somebody may be admitted next; with every place taken the queue just waits on
        if len(out.seqs) != len(s.running) or any(a is not b for a, b in zip(out.seqs, s.running)):
            return None
        limit = s.config.max_model_len
        for seq, n in zip(out.seqs, out.num_new_tokens):
            p = seq.params
            if (seq.status is not SequenceStatus.RUNNING or not seq.reaches_end(n) or p.presence_penalty != 0
                    or seq.num_output_tokens + 1 >= p.max_tokens or seq.num_tokens + 1 >= limit):  # fmt: skip
                return None
        if not can(out.seqs):
            return None
        for seq in out.seqs:
            if not s.manager.reserve(seq.cache, seq.num_tokens, 1):
                return None  # the scheduler decides who makes room, in its own turn
        return SchedulerOutput(seqs=list(out.seqs), num_new_tokens=[1] * len(out.seqs))

    def _drain_inbox(self, block: bool) -> None:
        while True:
            try:
                message = self._inbox.get(block=block)
            except queue.Empty:
                return
            block = False
            if message[0] == "add":
                _, seq, handle = message
                self._handles[seq.id] = handle
                self.num_prompt_tokens += seq.num_prompt_tokens
                self.scheduler.add(seq)
            elif message[0] == "abort":
                seq = self.scheduler.abort(message[1])
                if seq is not None:
                    self._close(seq)

    def _close(self, seq: Sequence, error: Optional[BaseException] = None) -> None:
        handle = self._handles.pop(seq.id)
        handle.num_cached_tokens = seq.num_cached_tokens
        self.num_cached_prompt_tokens += seq.num_cached_tokens
        handle.finished_at = time.perf_counter()
        self.runner.sampler.release(seq.id)
        handle._outbox.put(_Finished(seq.finish_reason or "error", error))

    def _loop(self) -> None:
        while not self._stopping:
            try:
                if not self.step():
                    self._drain_inbox(block=True)
            except Exception as error:  # fail the requests, keep the engine alive
                traceback.print_exc(file=sys.stderr)
                self._in_flight = None
                for seq in [*self.scheduler.running, *self.scheduler.waiting]:
                    self.scheduler.abort(seq.id)
                    seq.finish_reason = "error"
                    self._close(seq, error)


def create_engine(model, engine_config: EngineConfig, eos_token_ids=frozenset(), seed: Optional[int] = None) -> Engine:
    """Wire cache manager, pools, runner and scheduler around a loaded model (the thread is
    not started; reference atomserve/engine.py:237-264)."""
    manager = CacheManager(model.cache_requests(), engine_config.block_size, engine_config.num_blocks,
                           engine_config.max_num_seqs)  # fmt: skip
    runner = ModelRunner(model, manager)
    if runner.device.type == "cuda":
        ops.tune_library_rows(engine_config.max_num_batched_tokens)  # what a step with a prompt's portion brings
    return Engine(runner, Scheduler(engine_config, eos_token_ids, manager), seed=seed)

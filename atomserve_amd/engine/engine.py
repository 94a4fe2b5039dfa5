"""The engine: a pipeline of steps between the clients' queues and the GPU.

A step passes three stages, and one record (`_Flight`) carries it through them:

    plan    the scheduler says who runs and with how many tokens (`Scheduler.schedule`, or
            `Scheduler.plan_ahead` for the step after one that is still on the GPU)
    launch  the runner puts the pass and the sampling on the GPU and returns without waiting
    retire  the tokens are read, the scheduler takes them in, and each goes to its request

Up to two steps are under way: while the running requests do nothing but decode, the next
step is planned and launched before this one is retired (the GPU hands the sampled tokens to
it by itself), so the host's share of a step hides behind the GPU's.  A runner that has no
`launch` (a fake in tests) is simply run in the launch stage.

Clients on any thread reach the engine through one mailbox (requests and aborts) and get
their tokens back through one stream per request; the engine's own state is touched by one
thread only, the one that calls `step` (`start` makes a thread that does).  The engine deals
in token ids only.  Public interface and meanings of the counters follow the reference
(atomserve/engine.py:41-264).
"""

import itertools
import queue
import random
import sys
import threading
import time
import traceback
from collections import deque
from typing import Optional

from atomserve_amd.cache.manager import CacheManager
from atomserve_amd.config.engine_config import EngineConfig
from atomserve_amd.engine.runner import ModelRunner
from atomserve_amd.engine.scheduler import Scheduler, StepPlan
from atomserve_amd.engine.sequence import SamplingParams, Sequence, SequenceStatus

_END = object()  # last item of a request's stream


class RequestHandle:
    """A client's view of its request: iterating yields the token ids as they are made and ends
    when the request does; then `finish_reason` ("stop", "length", "abort" or "error") and the
    timing fields are final.  A request that an engine failure ended raises RuntimeError."""

    def __init__(self, request_id: int, engine: "Engine", num_prompt_tokens: int):
        self.id = request_id
        self.num_prompt_tokens = num_prompt_tokens
        self.num_output_tokens = 0
        self.num_cached_tokens = 0  # prompt tokens found in the prefix cache
        self.finish_reason: Optional[str] = None
        self.submitted_at = time.perf_counter()
        self.first_token_at: Optional[float] = None
        self.finished_at: Optional[float] = None
        self._engine = engine
        self._stream: queue.SimpleQueue = queue.SimpleQueue()  # lists of tokens, then (_END, reason, error)

    def __iter__(self):
        while True:
            item = self._stream.get()
            if isinstance(item, tuple) and item[0] is _END:
                _, self.finish_reason, error = item
                if error is not None:
                    raise RuntimeError("engine step failed") from error
                return
            yield from item

    def abort(self) -> None:
        self._engine.abort(self.id)

    @property
    def ttft(self) -> Optional[float]:
        """Seconds between submission and the first token."""
        if self.first_token_at is None:
            return None
        return self.first_token_at - self.submitted_at

    @property
    def decode_tokens_per_s(self) -> Optional[float]:
        """Rate of the tokens after the first; None before the end or for replies of one token."""
        if self.finished_at is None or self.first_token_at is None or self.num_output_tokens < 2:
            return None
        return (self.num_output_tokens - 1) / max(self.finished_at - self.first_token_at, 1e-9)

    # engine side
    def _deliver(self, tokens: list, now: float) -> None:
        if self.first_token_at is None:
            self.first_token_at = now
        self.num_output_tokens += len(tokens)
        self._stream.put(list(tokens))

    def _end(self, seq: Sequence, error: Optional[BaseException]) -> None:
        self.num_cached_tokens = seq.num_cached_tokens
        self.finished_at = time.perf_counter()
        self._stream.put((_END, seq.finish_reason or "error", error))


class _Flight:
    """A step between launch and retirement."""

    __slots__ = ("plan", "pending")

    def __init__(self, plan: StepPlan, pending):
        self.plan, self.pending = plan, pending


class _Ready:
    """What a runner without `launch` leaves behind: results that are there already."""

    device_tokens = None

    def __init__(self, results):
        self._results = results

    def results(self):
        return self._results


class Engine:
    MAX_IN_FLIGHT = 2

    def __init__(self, runner, scheduler: Scheduler, seed: Optional[int] = None):
        self.runner = runner
        self.scheduler = scheduler
        self.run_ahead = True  # False: every step is retired before the next is planned
        self._mail: queue.SimpleQueue = queue.SimpleQueue()  # ("submit", seq, handle) | ("abort", id) | ("wake",)
        self._open: dict = {}  # request id -> handle, until the request ends
        self._next_id = itertools.count()
        self._seeds = random.Random(seed)  # for requests that bring no seed of their own
        self._flights: deque = deque()
        self._thread: Optional[threading.Thread] = None
        self._halt = threading.Event()
        self._phases = None
        self.counters = dict.fromkeys(
            ("steps", "last_batch_seqs", "last_batch_tokens", "prompt_tokens", "cached_prompt_tokens",
             "generated_tokens", "preemptions"), 0)  # fmt: skip

    # ---- clients (any thread) ---------------------------------------------------------------
    def submit(self, prompt_ids, params: SamplingParams) -> RequestHandle:
        ids = [int(t) for t in prompt_ids]
        longest = self.scheduler.config.max_model_len
        if not ids or len(ids) >= longest:
            raise ValueError(f"prompt has {len(ids)} tokens; must be 1 to {longest - 1}")
        params.validated()
        vocab = getattr(self.runner, "vocab_size", None)
        if vocab is not None and (min(ids) < 0 or max(ids) >= vocab):
            raise ValueError(f"prompt holds a token id outside the vocabulary of {vocab}")
        seq = Sequence(next(self._next_id), ids, params)
        if params.seed is None:
            seq.noise_seed = self._seeds.getrandbits(63)
        handle = RequestHandle(seq.id, self, len(ids))
        self._mail.put(("submit", seq, handle))
        return handle

    def abort(self, request_id: int) -> None:
        self._mail.put(("abort", request_id))

    def generate(self, prompts, params: SamplingParams) -> list:
        """Runs the prompts to their ends on the calling thread and returns their replies.  All are
        submitted before the first step, so they share batches (reference atomserve/engine.py:137-146)."""
        handles = [self.submit(p, params) for p in prompts]
        while self.step():
            pass
        return [list(h) for h in handles]

    def start(self) -> None:
        """Serve on a thread of the engine's own until `shutdown`."""
        self._halt.clear()
        self._thread = threading.Thread(target=self._serve, name="atomserve-amd-engine", daemon=True)
        self._thread.start()

    def shutdown(self) -> None:
        self._halt.set()
        self._mail.put(("wake",))
        if self._thread is not None:
            self._thread.join()
            self._thread = None

    def warm_up(self) -> int:
        """Before serving: the decode steps of every batch size up to max_num_seqs (and every context
        length up to max_model_len, if that many graphs are kept) are captured now (kernels are compiled
        and loaded, the library's candidates tried) rather than at their first use.  Returns the number
        of graphs captured; 0 where decode steps run uncaptured."""
        tune = getattr(self.runner, "tune_prompt_lengths", None)
        if tune is not None:  # and the library's products of prompts of a few lengths, up to a step's budget
            tune(self.scheduler.config.max_num_batched_tokens)
        graphs = getattr(self.runner, "decode_graphs", None)
        if graphs is None:
            return 0
        return graphs.capture_ahead(self.scheduler.config.max_num_seqs, self.scheduler.config.max_model_len)

    def profile_phases(self, on: bool = True):
        """Starts (or ends) the split of the host's time by phase; returns the `PhaseTimes` that
        collects it.  While it is on no step is launched ahead, so that the wait for the GPU shows
        as what it is."""
        from atomserve_amd.engine.runner import PhaseTimes

        self._phases = PhaseTimes() if on else None
        if hasattr(self.runner, "phases"):
            self.runner.phases = self._phases
        return self._phases

    def stats(self) -> dict:
        manager = self.scheduler.manager
        total = manager.num_blocks
        used = total - manager.num_free
        report = {
            "running": len(self.scheduler.running),
            "waiting": len(self.scheduler.waiting),
            "kv_blocks_used": used,
            "kv_blocks_total": total,
            "kv_usage": used / total,
            "kv_blocks_cached": manager.num_cached,
        }
        report.update(self.counters)
        held = getattr(self.runner, "graph_bytes", None)
        if held is not None:
            report["graph_bytes"] = held()
        model = getattr(self.runner, "model", None)
        if model is not None:  # the weights, and their second copies in the order the decode kernels read them
            report["weight_bytes"] = model.num_weight_bytes
            report["stream_copy_bytes"] = model.num_stream_copy_bytes
        return report

    @property
    def steps_in_flight(self) -> int:
        return len(self._flights)

    # counters under the names they had as attributes
    num_steps = property(lambda self: self.counters["steps"])
    last_batch_seqs = property(lambda self: self.counters["last_batch_seqs"])
    last_batch_tokens = property(lambda self: self.counters["last_batch_tokens"])
    num_generated_tokens = property(lambda self: self.counters["generated_tokens"])
    num_preemptions = property(lambda self: self.counters["preemptions"])

    # ---- the pipeline (one thread) ----------------------------------------------------------
    def step(self) -> bool:
        """Retires one step, launching what the pipeline needs before; False when there is nothing to
        do.  If a stage raises, nothing stays in flight."""
        self._read_mail(wait=False)
        phases = self._phases
        try:
            if not self._flights:
                if not self.scheduler.has_work:
                    return False
                if phases is not None:
                    phases.begin()
                plan = self.scheduler.schedule()
                if not plan.seqs:
                    raise RuntimeError("scheduler has work but scheduled nothing")
                if phases is not None:
                    phases.mark("schedule")
                self._launch(plan, after=None)
            if len(self._flights) < self.MAX_IN_FLIGHT and phases is None:
                self._launch_ahead(self._flights[-1])
            self._retire(self._flights.popleft())
            if phases is not None:
                phases.mark("update")
                phases.steps += 1
        except BaseException:
            self._flights.clear()
            raise
        return True

    def _launch(self, plan: StepPlan, after) -> None:
        launch = getattr(self.runner, "launch", None)
        if launch is None:
            pending = _Ready(self.runner.execute(plan))
        else:
            pending = launch(plan, after=after.pending if after is not None else None)
        self._flights.append(_Flight(plan, pending))

    def _launch_ahead(self, head: _Flight) -> None:
        """Plans and launches the decode step after `head` if it is certain already: the scheduler says
        so, no message waits that could change who runs, no request needs its tokens on the host
        before the next sampling (a presence penalty does), and the runner can feed a step from the
        GPU's own tokens."""
        can = getattr(self.runner, "can_run_ahead", None)
        if not self.run_ahead or can is None or not self._mail.empty():
            return
        if any(seq.params.presence_penalty != 0 for seq in head.plan.seqs) or not can(head.plan.seqs):
            return
        plan = self.scheduler.plan_ahead(head.plan)
        if plan is not None:
            self._launch(plan, after=head)

    def _retire(self, flight: _Flight) -> None:
        results = flight.pending.results()
        gained = self.scheduler.update(flight.plan, results)
        now = time.perf_counter()
        c = self.counters
        c["steps"] += 1
        c["preemptions"] += len(flight.plan.preempted)
        c["last_batch_seqs"], c["last_batch_tokens"] = len(flight.plan.seqs), flight.plan.num_tokens
        for seq, tokens in gained:
            c["generated_tokens"] += len(tokens)
            self._open[seq.id]._deliver(tokens, now)
            if seq.status is SequenceStatus.FINISHED:
                self._close(seq)

    def _close(self, seq: Sequence, error: Optional[BaseException] = None) -> None:
        handle = self._open.pop(seq.id)
        self.counters["cached_prompt_tokens"] += seq.num_cached_tokens
        self.runner.sampler.release(seq.id)
        handle._end(seq, error)

    def _read_mail(self, wait: bool) -> None:
        """Takes in every message that is there; with `wait`, sleeps until there is one."""
        while True:
            try:
                message = self._mail.get(block=wait)
            except queue.Empty:
                return
            wait = False
            kind = message[0]
            if kind == "submit":
                _, seq, handle = message
                self._open[seq.id] = handle
                self.counters["prompt_tokens"] += seq.num_prompt_tokens
                self.scheduler.add(seq)
            elif kind == "abort":
                seq = self.scheduler.abort(message[1])
                if seq is not None:
                    self._close(seq)

    def _serve(self) -> None:
        while not self._halt.is_set():
            try:
                if not self.step():
                    self._read_mail(wait=True)
            except Exception as error:
                # the requests that were under way fail with the error; the thread goes on serving
                traceback.print_exc(file=sys.stderr)
                self._fail_all(error)

    def _fail_all(self, error: BaseException) -> None:
        self._flights.clear()
        for seq in list(self.scheduler.running) + list(self.scheduler.waiting):
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
        model.env.products.tune_rows(engine_config.max_num_batched_tokens)  # what a step with a prompt's portion brings
    return Engine(runner, Scheduler(engine_config, eos_token_ids, manager), seed=seed)

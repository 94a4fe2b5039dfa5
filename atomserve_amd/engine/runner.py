"""The step function: "run these tokens of these requests" as one pass over the GPU
(reference atomserve/runner.py:59-212).

`ModelRunner.step(rows)` runs exactly the tokens it is given, as one batch, from the
cache that earlier steps left, writes their keys and values, and returns the logits at
the wanted places.  It never changes a sequence: advancing and appending is the
scheduler's work, so the same plan can be inspected or retried.
"""

import gc
from collections import OrderedDict

import torch

from atomserve_amd.cache.manager import CacheManager
from atomserve_amd.cache.pools import CachePools
from atomserve_amd.engine.batch import Row, Staging, StepBatch
from atomserve_amd.engine.sequence import StepResult
from atomserve_amd.kernels import ops
from atomserve_amd.sampling.sampler import Sampler


def rows_for(seqs, num_new_tokens) -> list:
    """The usual rows: each sequence's next uncomputed tokens, logits at its last token only
    if that is its last known token (reference atomserve/runner.py:59-68)."""
    rows = []
    for seq, n in zip(seqs, num_new_tokens, strict=True):
        start = seq.num_computed_tokens
        if n < 1 or start + n > seq.num_tokens:
            raise ValueError(f"cannot run tokens {start}:{start + n} of {seq.num_tokens}")
        want = [n - 1] if seq.reaches_end(n) else []
        rows.append(Row(seq.token_ids[start : start + n], start, seq.cache.tables, want, seq.cache.state_slot))
    return rows


class PhaseTimes:
    """Where the host's time of a step goes: seconds per phase, summed over steps.  The engine and the
    runner call `mark(phase)` at the end of each phase when one of these is installed
    (`Engine.profile_phases`); the phases are those of the reference's bench/engine.py:129-171:
    schedule, pack (rows, flat integers, upload), launch (the pass put on the GPU), sample (the
    sampling kernels put on the GPU), wait (for the GPU), update (tokens taken in and handed out)."""

    PHASES = ("schedule", "pack", "launch", "sample", "wait", "update")

    def __init__(self):
        import time

        self._now = time.perf_counter
        self.seconds = dict.fromkeys(self.PHASES, 0.0)
        self.steps = 0
        self._last = self._now()

    def begin(self) -> None:
        self._last = self._now()

    def mark(self, phase: str) -> None:
        now = self._now()
        self.seconds[phase] += now - self._last
        self._last = now

    def mean_us(self) -> dict:
        return {k: round(v / max(1, self.steps) * 1e6, 1) for k, v in self.seconds.items()}


_capture_primer = None  # a trivial captured graph that lives as long as the process


def _prime_capture(device) -> None:
    """Once per process, before the first capture under inference mode: a trivial capture outside it,
    kept alive.  torch keeps the random generator's state for captures in tensors that it makes when
    the first graph of the process registers (and drops when the last one is destroyed) and fills in
    place at every capture; made under inference mode they would refuse that update in a later capture
    outside it (a caller's own graphs, after this engine's).  While this graph lives they stay as they
    were made here."""
    global _capture_primer
    if _capture_primer is not None:
        return
    with torch.inference_mode(False):
        scratch = torch.zeros(1, device=device)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            scratch += 1
    _capture_primer = (graph, scratch)


def _bucket(n: int, steps) -> int:
    for s in steps:
        if n <= s:
            return s
    return 0


class DecodeGraphs:
    """Decode steps (every row brings one token) replayed as HIP graphs.

    A decode step is some hundred small launches; issuing them from the host costs more than
    running them.  For each (rows rounded up, context rounded up) one pass is captured; later
    steps copy their integers into the captured step's buffer and replay it.  Rows that pad a
    step to its bucket store nothing and their logits are dropped.  Up to 16 rows every captured
    kernel is this package's; above, the matrix products are the library's, which replay
    correctly (checked against eager steps in the tests, several replays with eager work between).

    A step is captured on rows that pad only (they store nothing and use the state slot that belongs
    to nobody), so capturing, and the runs that warm it up, touch no request's cache or state; the
    real rows are packed into the captured buffer afterwards.  A model whose mixers keep a state of
    their own replays like any other if all its parts say they are capturable.

    All captured steps draw their intermediate tensors from one memory pool and write their logits
    into one buffer [largest bucket, vocab] (they never run at the same time; a step's logits are
    read, by the sampling kernels or a copy, before the next step of the same stream overwrites
    them); at most `MAX_GRAPHS` are kept, the one replayed longest ago goes first.  `bytes_held`
    is the memory the captures took from the device."""

    ROW_BUCKETS = (1, 2, 4, 8, 16, 32, 48, 64, 96, 128, 192, 256)
    CONTEXT_STEP = 1024
    MAX_GRAPHS = 64

    def __init__(self, runner):
        self.runner = runner
        self.graphs = OrderedDict()  # (rows, context) -> (graph, its batch, its logits), least recently used first
        self.pool = None
        self.filler_tables = [[0] for _ in runner.manager.paged_groups]  # one object: a filler row is recognised
        self.logits = None  # [most_rows, vocab] fp32, shared by all captured steps
        self.most_rows = _bucket(min(self.ROW_BUCKETS[-1], runner.manager.max_num_seqs), self.ROW_BUCKETS)
        self.bytes_held = 0

    def filler(self) -> Row:
        """A row that pads a step: one token at position 0 that stores nothing; if the model keeps
        per-request state, it works on the slot that belongs to nobody."""
        slot = self.runner.pools.scrap_slot if self.runner.manager.state_groups else -1
        return Row([0], 0, self.filler_tables, [0], slot, store=False)

    def eligible(self, rows) -> bool:
        r = self.runner
        return (
            r.device.type == "cuda"
            and r.model.capturable
            and 0 < len(rows) <= self.most_rows
            and all(len(row.tokens) == 1 for row in rows)
        )

    def run(self, rows, tokens_from=None):
        """tokens_from: int32 [len(rows)] on the GPU, the rows' tokens where the host does not know them
        yet (the step before is still running); copied into the step's buffer after the host's integers."""
        r = self.runner
        bs = r.manager.block_size
        n = _bucket(len(rows), self.ROW_BUCKETS)
        longest = max(row.start + 1 for row in rows)
        context = -(-longest // self.CONTEXT_STEP) * self.CONTEXT_STEP
        width = -(-context // bs)
        # every row of the captured step yields logits; rows that want none are dropped after the replay
        padded = [row if row.want else Row(row.tokens, row.start, row.tables, [0], row.state_slot) for row in rows]
        padded += [self.filler() for _ in range(n - len(rows))]
        key = (n, context)
        entry = self.graphs.get(key)
        if entry is None:
            while len(self.graphs) >= self.MAX_GRAPHS:
                self.graphs.popitem(last=False)
            entry = self.graphs[key] = self._capture(n, width, context)
            fresh = True
        else:
            self.graphs.move_to_end(key)
            fresh = False
        if fresh or not entry[1].advance(padded):
            # other requests than last time, or a window moved: pack anew into the captured buffer
            batch = r.prepare(padded, table_width=width, max_context=context, into=entry[1])
            entry = self.graphs[key] = (entry[0], batch, entry[2])
        if tokens_from is not None:
            entry[1].token_ids[: len(rows)].copy_(tokens_from)
        graph, batch, logits = entry
        if r.phases is not None:
            r.phases.mark("pack")
        graph.replay()
        wanted = [i for i, row in enumerate(rows) if row.want]
        if wanted == list(range(len(rows))):
            return logits[: len(rows)]
        return logits[torch.tensor(wanted, dtype=torch.long, device=logits.device)] if wanted else logits[:0]


    def _capture(self, n: int, width: int, context: int):
        """Captures the decode step of `n` rows and contexts up to `context`, on padding rows."""
        r = self.runner
        before = torch.cuda.memory_reserved()
        if self.logits is None:
            self.logits = torch.empty((self.most_rows, r.vocab_size), dtype=torch.float32, device=r.device)
        batch = r.prepare([self.filler() for _ in range(n)], table_width=width, max_context=context)
        out = self.logits[:n]
        products = r.model.env.products
        products.tune_rows(n)  # a bucket's products come again at every replay: worth trying the library's candidates
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            r.model.forward(batch, logits=out)  # loads every library and warms the allocator before capture
            for _ in range(3):  # and while the library's products are still being tried, again
                if not products.trials_pending():
                    break
                r.model.forward(batch, logits=out)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        products.settle()  # what the warm-up tried among the library's products is decided now
        batch.shared.clear()  # what parts computed once for the warm-up must be computed in the graph too
        _prime_capture(r.device)
        graph = torch.cuda.CUDAGraph()
        if self.pool is None:
            self.pool = torch.cuda.graph_pool_handle()
        # No garbage collection while the stream is capturing: a collected object of an
        # earlier engine (a graph, a tensor) would be destroyed in the middle of the capture,
        # which the runtime answers by aborting the process.
        gc.collect()
        collecting = gc.isenabled()
        gc.disable()
        try:
            with torch.cuda.graph(graph, pool=self.pool):
                r.model.forward(batch, logits=out)
        finally:
            if collecting:
                gc.enable()
        self.bytes_held = self._bytes_now(self.bytes_held + max(0, torch.cuda.memory_reserved() - before))
        return graph, batch, out

    def _bytes_now(self, otherwise: int) -> int:
        """The shared logits plus the segments of the captures' memory pool (which nothing else can use
        while the graphs live); `otherwise` where the allocator does not tell segments by pool."""
        held = self.logits.numel() * self.logits.element_size()
        segments = torch.cuda.memory_snapshot()
        if not segments or "segment_pool_id" not in segments[0]:
            return otherwise
        return held + sum(s["total_size"] for s in segments if tuple(s["segment_pool_id"]) == tuple(self.pool))

    @torch.inference_mode()
    def capture_ahead(self, max_rows: int, max_context: int = 0) -> int:
        """Captures the decode step of every row bucket up to the one that holds `max_rows`, with rows that
        store nothing: a server does this once at its start instead of pausing (for tens of milliseconds)
        when a bucket is first met.  For every context bucket up to `max_context` if all of them fit among
        the graphs that are kept, else for the first one only.  Returns how many graphs were captured."""
        if not self.eligible([self.filler()]):
            return 0
        before = len(self.graphs)
        most = min(max_rows, self.most_rows)
        row_buckets = [n for n in self.ROW_BUCKETS if n < most] + [_bucket(most, self.ROW_BUCKETS)]
        contexts = [self.CONTEXT_STEP * i for i in range(1, -(-max(max_context, 1) // self.CONTEXT_STEP) + 1)]
        if len(contexts) * len(row_buckets) > self.MAX_GRAPHS:
            contexts = contexts[:1]
        bs = self.runner.manager.block_size
        for context in contexts:
            for n in row_buckets:
                if (n, context) not in self.graphs:
                    self.graphs[(n, context)] = self._capture(n, -(-context // bs), context)
        return len(self.graphs) - before


class PendingStep:
    """A step that is on the GPU, sampling included; `results()` waits for its tokens."""

    def __init__(self, samples, num_computed, device_tokens, host_tokens, event, phases=None):
        self.phases = phases
        self.samples = samples  # per scheduled sequence: whether the step gives it a token
        self.num_computed = num_computed  # per scheduled sequence: its leading tokens in the cache afterwards
        self.device_tokens = device_tokens  # int32 on the GPU, one per sampling sequence, or None
        self.host_tokens = host_tokens  # pinned; filled when `event` has passed
        self.event = event

    def results(self) -> list:
        tokens = iter(())
        if self.device_tokens is not None:
            self.event.synchronize()
            if self.phases is not None:
                self.phases.mark("wait")
            tokens = iter(self.host_tokens[: self.device_tokens.shape[0]].tolist())
        return [StepResult([next(tokens)] if yes else [], n) for yes, n in zip(self.samples, self.num_computed)]


class ModelRunner:
    """Owns the model, the cache pools and the sampler; executes one step for a list of rows."""

    def __init__(self, model, manager: CacheManager, pools: CachePools = None, use_graphs: bool = True):
        self.model = model
        self.manager = manager
        self.device = model.env.device
        self.pools = pools if pools is not None else CachePools(manager, model.env.dtype, self.device)
        self.sampler = Sampler(self.device)
        self.staging = Staging(self.device)
        self.vocab_size = model.plan.vocab_size
        self.row_splits = model.row_splits()  # how the model's mixers want the rows of a step sorted
        self.decode_graphs = DecodeGraphs(self) if use_graphs else None
        self._token_buffers = []  # pinned, used in turn: the sampled tokens of the steps on their way
        self._token_turn = 0
        self.phases = None  # a PhaseTimes while the host's time is being split up

    def prepare(self, rows, **layout) -> StepBatch:
        return StepBatch(rows, self.manager.block_size, len(self.manager.paged_groups), self.vocab_size,
                         self.device, pools=self.pools, staging=self.staging, row_splits=self.row_splits,
                         **layout)  # fmt: skip

    @torch.inference_mode()
    def step(self, rows, tokens_from=None) -> torch.Tensor:
        """Logits [sum of len(row.want), vocab] fp32, in the order of the rows and of `want`.
        tokens_from: see `DecodeGraphs.run`; for decode steps that are replayed only."""
        if self.decode_graphs is not None and self.decode_graphs.eligible(rows):
            if any(w != 0 for row in rows for w in row.want):
                raise ValueError("a row wants logits at a place outside its tokens")
            return self.decode_graphs.run(rows, tokens_from)
        if tokens_from is not None:
            raise ValueError("only a replayed decode step takes its tokens from the GPU")
        batch = self.prepare(rows)
        if self.phases is not None:
            self.phases.mark("pack")
        return self.model.forward(batch)

    @torch.inference_mode()
    def run(self, seqs, num_new_tokens) -> torch.Tensor:
        """One step for sequences; row j of the result belongs to the j-th sequence that
        reaches its end this step (reference atomserve/runner.py:182-192)."""
        return self.step(rows_for(seqs, num_new_tokens))

    def execute(self, out) -> list:
        """Run one scheduled step and sample: a sequence that reaches the end of its known
        tokens gets one new token (reference atomserve/runner.py:194-212)."""
        return self.launch(out).results()

    def can_run_ahead(self, seqs) -> bool:
        """Whether a decode step of these sequences can go to the GPU before the step before it has been
        read: it must be a replayed step, whose token buffer the GPU can fill itself."""
        graphs = self.decode_graphs
        return graphs is not None and graphs.eligible([graphs.filler()] * len(seqs))

    @torch.inference_mode()
    def tune_prompt_lengths(self, most_tokens: int) -> list:
        """Runs a prompt that stores nothing at each of a few lengths (128, 192, 256, 384, ... up to `most_tokens`)
        until the library's candidates for its products have been tried and the fastest chosen; prompts
        of other lengths then take what the next length above them chose.  Returns the lengths run."""
        products = self.model.env.products
        if self.device.type != "cuda" or products.fixed:
            return []
        bs, lengths, n = self.manager.block_size, [], 128
        while n <= most_tokens:
            lengths.extend(m for m in (n, n + n // 2) if m <= most_tokens)
            n *= 2
        slot = self.pools.scrap_slot if self.manager.state_groups else -1
        for n in lengths:
            products.tune_rows(n)
            tables = [[0] * -(-n // bs) for _ in self.manager.paged_groups]
            rows = [Row([0] * n, 0, tables, [n - 1], slot, store=False)]
            for _ in range(4):
                self.step(rows)
                if not products.trials_pending():
                    break
            products.settle()
        if lengths:
            ops.prepare_library_adoption()
        torch.cuda.synchronize()
        return lengths

    def graph_bytes(self) -> int:
        """Device memory that captured decode steps hold (their shared logits and memory pool)."""
        return 0 if self.decode_graphs is None else self.decode_graphs.bytes_held

    @torch.inference_mode()
    def launch(self, out, after: PendingStep = None) -> PendingStep:
        """Put one scheduled step on the GPU, sampling included, without waiting for it.

        after: the step before it, not read yet, when this one runs ahead.  Then every sequence decodes
        the token that `after` samples for it, which the GPU hands over itself, at the position after its
        last known token; the sequences' own bookkeeping is one step behind until `after` is read."""
        if after is None:
            samples = [s.reaches_end(n) for s, n in zip(out.seqs, out.num_new_tokens, strict=True)]
            num_computed = [s.num_computed_tokens + n for s, n in zip(out.seqs, out.num_new_tokens)]
            logits = self.step(rows_for(out.seqs, out.num_new_tokens))
        else:
            samples = [True] * len(out.seqs)
            num_computed = [s.num_tokens + 1 for s in out.seqs]
            rows = [Row([0], s.num_tokens, s.cache.tables, [0], s.cache.state_slot) for s in out.seqs]
            logits = self.step(rows, tokens_from=after.device_tokens)
        if self.phases is not None:
            self.phases.mark("launch")
        sampling = [s for s, yes in zip(out.seqs, samples) if yes]
        device_tokens = self.sampler.launch(logits, sampling, ahead=0 if after is None else 1)
        host_tokens = event = None
        if device_tokens is not None:
            # three pinned buffers in turn: at most two steps are on their way at any time
            if len(self._token_buffers) < 3:
                self._token_buffers.append(torch.empty(4096, dtype=torch.int32, pin_memory=True))
            self._token_turn = (self._token_turn + 1) % len(self._token_buffers)
            host_tokens = self._token_buffers[self._token_turn]
            if host_tokens.numel() < device_tokens.shape[0]:
                host_tokens = self._token_buffers[self._token_turn] = torch.empty(
                    device_tokens.shape[0], dtype=torch.int32, pin_memory=True)  # fmt: skip
            host_tokens[: device_tokens.shape[0]].copy_(device_tokens, non_blocking=True)
            event = torch.cuda.Event()
            event.record()
        if self.phases is not None:
            self.phases.mark("sample")
        return PendingStep(samples, num_computed, device_tokens, host_tokens, event, self.phases)

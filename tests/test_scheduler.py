"""The scheduler's decisions, without a model or a GPU.

A fake runner simulates the cache slot by slot: it "writes" each scheduled token into
the slot its block table points to and predicts the next token from what it reads
back, so a page given to two requests, a missing recomputation after preemption, a
wrong prefix hit or a short block table all change the outputs (the method of
reference tests/test_scheduler.py:20-92; the policy vectors cite their lines)."""

import pytest

from atomserve_amd.config import EngineConfig
from atomserve_amd.engine.batch import slot_of
from atomserve_amd.engine.scheduler import Scheduler
from atomserve_amd.engine.sequence import SamplingParams, Sequence, SequenceStatus, StepResult

EOS = 999


def table_of(seq) -> list:
    """The request's block table in the one group of pages these schedulers have."""
    return seq.cache.tables[0] if seq.cache.tables else []

GREEDY = SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True)


class FakeRunner:
    def __init__(self, block_size):
        self.bs, self.slots = block_size, {}

    def execute(self, out):
        results = []
        for seq, n in zip(out.seqs, out.num_new_tokens, strict=True):
            start, end = seq.num_computed_tokens, seq.num_computed_tokens + n
            assert end <= len(table_of(seq)) * self.bs, "block table too small"
            for p in range(start, end):
                self.slots[slot_of(table_of(seq), p, self.bs)] = seq.token_ids[p]
            tokens = []
            if seq.reaches_end(n):
                context = [self.slots[slot_of(table_of(seq), p, self.bs)] for p in range(end)]
                tokens.append(sum((i + 1) * t for i, t in enumerate(context)) % 500)
            results.append(StepResult(tokens, end))
        return results


def make(**config):
    cfg = {"block_size": 4, "num_blocks": 64, "max_model_len": 64, **config}
    return Scheduler(EngineConfig(**cfg), frozenset({EOS})), FakeRunner(cfg["block_size"])


def sharing_is_safe(s):
    bs, owners = s.config.block_size, {}
    for seq in s.running:
        for i, page in enumerate(table_of(seq)):
            owners.setdefault(page, []).append((seq, i))
    for sharers in owners.values():
        if len(sharers) > 1:
            assert len({i for _, i in sharers}) == 1, "shared at different positions"
            assert all((i + 1) * bs <= q.num_computed_tokens for q, i in sharers), "shared before it was computed"


def drive(s, runner):
    preemptions = 0
    while s.has_work:
        out = s.schedule()
        assert out.seqs, "no progress"
        assert len(out.seqs) <= s.config.max_num_seqs and out.num_tokens <= s.config.max_num_batched_tokens
        sharing_is_safe(s)
        preemptions += len(out.preempted)
        s.update(out, runner.execute(out))
        s.manager.check()
    assert s.manager.num_free == s.manager.num_blocks, "leaked pages"
    return preemptions


def run(prompts, params=GREEDY, **config):
    s, runner = make(**config)
    seqs = [Sequence(i, list(p), params) for i, p in enumerate(prompts)]
    for q in seqs:
        s.add(q)
    preemptions = drive(s, runner)
    return [q.output_ids for q in seqs], s, preemptions


PROMPTS = [[1, 2, 3], [4, 5, 6, 7, 8, 9, 10], [11], [12, 13, 14, 15, 16], [17, 18]]


def alone(prompt):
    return run([prompt])[0][0]


def test_batching_limits_and_queueing_do_not_change_outputs():
    expected = [alone(p) for p in PROMPTS]
    outputs, _, preemptions = run(PROMPTS)
    assert outputs == expected and preemptions == 0 and all(len(o) == 12 for o in outputs)
    assert run(PROMPTS, max_num_seqs=2, max_num_batched_tokens=16)[0] == expected
    assert run([[1] * 20, [2, 3], list(range(30, 47))], max_num_batched_tokens=8, max_num_seqs=4)[0] == [
        alone([1] * 20), alone([2, 3]), alone(list(range(30, 47)))]  # fmt: skip


def test_when_pages_run_out_the_newest_is_preempted_and_recomputed():
    """8 pages of 4 tokens hold 32 tokens; five requests growing to about 20 cannot all fit."""
    outputs, _, preemptions = run(PROMPTS, num_blocks=8, max_model_len=32)
    assert preemptions > 0 and outputs == [alone(p) for p in PROMPTS]


def test_preemption_evicts_the_newest_and_requeues_it_first():
    # reference tests/test_scheduler.py:121-135
    s = Scheduler(EngineConfig(block_size=4, num_blocks=2, max_model_len=8), frozenset())
    old, new = Sequence(0, [1, 2, 3], GREEDY), Sequence(1, [4, 5, 6], GREEDY)
    runner = FakeRunner(4)
    s.add(old)
    s.add(new)
    for _ in range(2):
        out = s.schedule()
        s.update(out, runner.execute(out))
    out = s.schedule()  # both need a second page; only one can grow
    assert out.preempted == [new] and out.seqs == [old]
    assert s.waiting[0] is new and new.status is SequenceStatus.WAITING
    assert new.num_computed_tokens == 0 and table_of(new) == []
    # nobody is admitted in a step that had to preempt
    assert len(s.running) == 1


def test_a_request_that_is_itself_the_newest_waits_instead_of_evicting_scheduled_ones():
    s = Scheduler(EngineConfig(block_size=4, num_blocks=3, max_model_len=12), frozenset())
    a, b = Sequence(0, [1] * 4, GREEDY), Sequence(1, [2] * 7, GREEDY)
    runner = FakeRunner(4)
    s.add(a)
    s.add(b)
    out = s.schedule()
    assert out.num_new_tokens == [4, 7]
    s.update(out, runner.execute(out))
    out = s.schedule()  # a needs page 2 of its own: the newest (b) goes, a runs
    assert out.seqs == [a] and out.preempted == [b]


def test_admission_respects_the_token_budget_in_order():
    # reference tests/test_scheduler.py:138-149
    s = Scheduler(EngineConfig(block_size=4, num_blocks=64, max_model_len=64, max_num_batched_tokens=8, max_num_seqs=4))
    for i, prompt in enumerate([[1] * 5, [2] * 3, [3] * 2]):
        s.add(Sequence(i, prompt, GREEDY))
    out = s.schedule()
    assert out.num_new_tokens == [5, 3] and len(s.waiting) == 1


def test_long_prompt_runs_in_portions_beside_decodes():
    # reference tests/test_scheduler.py:152-170: budget 8, one decode + a 20-token prompt -> 7, 7, 6
    s, runner = make(max_num_batched_tokens=8, max_num_seqs=4)
    short, long = Sequence(0, [2, 3], GREEDY), Sequence(1, [1] * 20, GREEDY)
    s.add(short)
    out = s.schedule()
    s.update(out, runner.execute(out))
    s.add(long)
    plans = []
    while long.num_computed_tokens < long.num_prompt_tokens:
        out = s.schedule()
        plans.append(list(zip(out.seqs, out.num_new_tokens)))
        s.update(out, runner.execute(out))
    assert plans == [[(short, 1), (long, 7)], [(short, 1), (long, 7)], [(short, 1), (long, 6)]]
    assert len(long.output_ids) == 1


def test_finish_reasons():
    # reference tests/test_scheduler.py:179-201
    s = Scheduler(EngineConfig(block_size=4, num_blocks=16, max_model_len=16), frozenset({7}))
    stops = Sequence(0, [1], SamplingParams(temperature=0.0, max_tokens=5))
    ignores = Sequence(1, [1], SamplingParams(temperature=0.0, max_tokens=3, ignore_eos=True))
    too_long = Sequence(2, [1] * 14, SamplingParams(temperature=0.0, max_tokens=99, ignore_eos=True))
    for q in (stops, ignores, too_long):
        s.add(q)
    while s.has_work:
        out = s.schedule()
        s.update(out, [StepResult([7] if q.reaches_end(n) else [], q.num_computed_tokens + n)
                       for q, n in zip(out.seqs, out.num_new_tokens)])  # fmt: skip
    assert (stops.finish_reason, stops.output_ids) == ("stop", [7])
    assert (ignores.finish_reason, ignores.output_ids) == ("length", [7, 7, 7])
    assert (too_long.finish_reason, too_long.num_tokens) == ("length", 16)
    assert s.manager.num_free == 16


def test_abort_frees_running_and_waiting_requests():
    s = Scheduler(EngineConfig(block_size=4, num_blocks=16, max_model_len=16, max_num_seqs=1, max_num_batched_tokens=8))
    running, waiting = Sequence(0, [1, 2], GREEDY), Sequence(1, [3], GREEDY)
    s.add(running)
    s.add(waiting)
    s.schedule()
    assert running.status is SequenceStatus.RUNNING and table_of(running)
    assert s.abort(0) is running and s.abort(1) is waiting and s.abort(1) is None
    assert running.finish_reason == waiting.finish_reason == "abort"
    assert not s.has_work and s.manager.num_free == 16


def test_prefix_reuse_counts():
    # reference tests/test_scheduler.py:223-245, 287-303: 8 of 10, 4 of 8, 12 of 20
    s, runner = make()
    prompt = list(range(40, 50))
    first = Sequence(0, list(prompt), GREEDY)
    s.add(first)
    drive(s, runner)
    again = Sequence(1, list(prompt), GREEDY)
    s.add(again)
    drive(s, runner)
    assert (first.num_cached_tokens, again.num_cached_tokens) == (0, 8) and again.output_ids == first.output_ids

    s, runner = make()
    for i in range(2):
        q = Sequence(i, list(range(8)), GREEDY)
        s.add(q)
        drive(s, runner)
    assert q.num_cached_tokens == 4

    prompt = list(range(60, 80))
    s, runner = make(max_num_batched_tokens=14, max_num_seqs=4)
    a = Sequence(0, list(prompt), GREEDY)
    s.add(a)
    out = s.schedule()
    s.update(out, runner.execute(out))
    assert a.num_computed_tokens == 14
    s.abort(a.id)
    b = Sequence(1, list(prompt), GREEDY)
    s.add(b)
    drive(s, runner)
    assert b.num_cached_tokens == 12 and b.output_ids == alone(prompt)


def test_running_requests_share_a_prefix_and_pressure_keeps_outputs():
    system = list(range(100, 112))
    a, b = Sequence(0, system + [1, 2], GREEDY), Sequence(1, system + [3], GREEDY)
    s, runner = make()
    s.add(a)
    for _ in range(2):
        out = s.schedule()
        s.update(out, runner.execute(out))
    s.add(b)
    out = s.schedule()
    assert table_of(b)[:3] == table_of(a)[:3] and out.num_new_tokens == [1, 1]
    s.update(out, runner.execute(out))
    drive(s, runner)
    assert a.output_ids == alone(system + [1, 2]) and b.output_ids == alone(system + [3])

    shared = [7, 7, 7, 7, 8, 8, 8, 8]
    prompts = [shared + [i, i + 1] for i in range(6)]
    outputs, _, preemptions = run(prompts, num_blocks=10, max_model_len=40)
    assert preemptions > 0 and outputs == [alone(p) for p in prompts]


def test_prefix_caching_can_be_disabled():
    s, runner = make(enable_prefix_caching=False)
    for i in range(2):
        q = Sequence(i, list(range(10)), GREEDY)
        s.add(q)
        drive(s, runner)
    assert q.num_cached_tokens == 0 and s.manager.num_cached == 0


def test_windowed_model_gives_pages_back_while_decoding():
    from atomserve_amd.cache import CacheManager
    from atomserve_amd.parts.base import PagedCacheRequest

    cfg = EngineConfig(block_size=4, num_blocks=6, max_model_len=24)
    manager = CacheManager({0: PagedCacheRequest(1, 8, window=6)}, 4, 6, cfg.max_num_seqs)
    s = Scheduler(cfg, frozenset(), manager)
    q = Sequence(0, [1, 2, 3], SamplingParams(temperature=0.0, max_tokens=20, ignore_eos=True))
    s.add(q)
    most = 0
    while s.has_work:
        out = s.schedule()
        s.update(out, [StepResult([5] if x.reaches_end(n) else [], x.num_computed_tokens + n)
                       for x, n in zip(out.seqs, out.num_new_tokens)])  # fmt: skip
        most = max(most, manager.num_blocks - manager.num_free)
    assert q.num_tokens == 23 and most <= 3 and manager.num_free == 6  # 23 tokens never held more than 3 pages


@pytest.mark.parametrize("seed", range(12))
def test_random_arrivals_aborts_and_tight_pools_keep_every_output(seed):
    """Requests arrive while others run, some are aborted half-way, the pool is small enough to
    preempt, budgets and row limits are drawn at random, half of the prompts share a prefix: every
    request that finishes has the tokens it gets alone, nothing is shared unsafely at any step,
    and every page is back at the end."""
    import random

    rng = random.Random(seed)
    bs = rng.choice([2, 4, 8])
    longest = 40
    blocks = rng.randint(-(-longest // bs), 2 * -(-longest // bs))
    seqs_limit = rng.randint(1, 6)
    config = dict(block_size=bs, num_blocks=blocks, max_model_len=min(longest, blocks * bs), max_num_seqs=seqs_limit,
                  max_num_batched_tokens=rng.randint(seqs_limit, 24), enable_prefix_caching=rng.random() < 0.7)  # fmt: skip
    s, runner = make(**config)
    prefix = [rng.randrange(1, 400) for _ in range(2 * bs + 1)]
    arrivals = []
    for i in range(14):
        own = [rng.randrange(1, 400) for _ in range(rng.randint(1, 20))]
        prompt = (prefix + own)[: longest - 13] if rng.random() < 0.5 else own
        params = SamplingParams(temperature=0.0, max_tokens=rng.randint(1, 12), ignore_eos=True)
        arrivals.append((rng.randint(0, 12), Sequence(i, prompt, params)))
    aborts = {rng.randrange(14): rng.randint(1, 30) for _ in range(3)}  # request -> step at which it is aborted
    step, preemptions, aborted = 0, 0, set()
    while s.has_work or any(at >= step for at, _ in arrivals):
        for at, seq in arrivals:
            if at == step:
                s.add(seq)
        for victim, at in aborts.items():
            if at == step and s.abort(victim) is not None:
                aborted.add(victim)
        if s.has_work:
            out = s.schedule()
            assert out.seqs, "no progress"
            assert len(out.seqs) <= seqs_limit and out.num_tokens <= config["max_num_batched_tokens"]
            sharing_is_safe(s)
            preemptions += len(out.preempted)
            s.update(out, runner.execute(out))
            s.manager.check()
        step += 1
        assert step < 2000
    assert s.manager.num_free == blocks
    for _, seq in arrivals:
        if seq.id in aborted:
            assert seq.finish_reason == "abort"
            continue
        assert seq.finish_reason == "length"
        alone_out = run([seq.token_ids[: seq.num_prompt_tokens]], seq.params, block_size=bs)[0][0]
        assert seq.output_ids == alone_out, (seed, seq.id, preemptions)

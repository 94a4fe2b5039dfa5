"""The engine loop with a fake runner (no GPU): streaming, threads, abort, validation and
failure handling (reference atomserve/engine.py:109-234, tests/test_engine.py:52-96)."""

import threading
import time

import pytest

from atomserve_amd.config import EngineConfig
from atomserve_amd.engine.engine import Engine
from atomserve_amd.engine.scheduler import Scheduler
from atomserve_amd.engine.sequence import SamplingParams, StepResult

GREEDY = SamplingParams(temperature=0.0, max_tokens=10, ignore_eos=True)
PROMPTS = [[1, 2, 3], [4, 5, 6, 7, 8, 9, 10, 11], [12], [13, 14, 15, 16, 17], [18, 19]]


class _NoSampler:
    def release(self, seq_id):
        pass


class CountingRunner:
    """Next token = (sum of all known tokens) % 97: depends on the whole context."""

    vocab_size = 1000
    sampler = _NoSampler()
    fail_at = None
    delay = 0.0

    def __init__(self):
        self.calls = 0

    def execute(self, out):
        self.calls += 1
        if self.delay:
            time.sleep(self.delay)
        if self.fail_at is not None and self.calls >= self.fail_at:
            raise RuntimeError("device fell over")
        return [StepResult([sum(s.token_ids) % 97] if s.reaches_end(n) else [], s.num_computed_tokens + n)
                for s, n in zip(out.seqs, out.num_new_tokens)]  # fmt: skip


def engine(**kw):
    cfg = EngineConfig(**{"block_size": 4, "num_blocks": 64, "max_model_len": 64, **kw})
    return Engine(CountingRunner(), Scheduler(cfg, frozenset()))


def test_generate_batches_and_matches_each_prompt_alone():
    alone = [engine().generate([p], GREEDY)[0] for p in PROMPTS]
    assert engine().generate(PROMPTS, GREEDY) == alone
    assert engine(num_blocks=8, max_model_len=32).generate(PROMPTS, GREEDY) == alone
    e = engine(max_num_batched_tokens=4, max_num_seqs=4)
    assert e.generate(PROMPTS, GREEDY) == alone
    stats = e.stats()
    assert stats["generated_tokens"] == 50 and stats["prompt_tokens"] == 19 and stats["kv_blocks_used"] == 0


def test_engine_thread_serves_concurrent_clients():
    alone = [engine().generate([p], GREEDY)[0] for p in PROMPTS]
    e = engine()
    e.start()
    results = {}

    def client(i):
        handle = e.submit(PROMPTS[i], GREEDY)
        results[i] = list(handle)
        assert handle.finish_reason == "length" and handle.ttft is not None and handle.ttft >= 0

    threads = [threading.Thread(target=client, args=(i,)) for i in range(len(PROMPTS))]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=30)
    e.shutdown()
    assert [results[i] for i in range(len(PROMPTS))] == alone


def test_abort_stops_a_stream_and_frees_its_pages():
    e = engine()
    e.runner.delay = 0.005  # a step takes time, so the abort arrives while the request runs
    e.start()
    handle = e.submit([1, 2, 3], SamplingParams(temperature=0.0, max_tokens=50, ignore_eos=True))
    tokens = []
    for token in handle:
        tokens.append(token)
        if len(tokens) == 3:
            handle.abort()
    e.shutdown()
    assert handle.finish_reason == "abort" and 3 <= len(tokens) < 50
    assert e.stats()["kv_blocks_used"] == 0


def test_submit_validates():
    e = engine()
    with pytest.raises(ValueError, match="prompt"):
        e.submit([], GREEDY)
    with pytest.raises(ValueError, match="prompt"):
        e.submit([1] * 64, GREEDY)
    with pytest.raises(ValueError, match="max_tokens"):
        e.submit([1], SamplingParams(max_tokens=0))
    for bad, named in ((dict(temperature=-0.5), "temperature"), (dict(top_p=0.0), "top_p"), (dict(top_p=1.5), "top_p"),
                       (dict(top_k=-1), "top_k"), (dict(temperature=float("nan")), "temperature")):  # fmt: skip
        with pytest.raises(ValueError, match=named):
            e.submit([1], SamplingParams(**bad))
    with pytest.raises(ValueError, match="vocabulary"):
        e.submit([1, 1000], GREEDY)


def test_a_failing_step_fails_the_requests_and_keeps_the_engine_alive():
    e = engine()
    e.runner.fail_at = 3
    e.start()
    handle = e.submit([1, 2, 3], GREEDY)
    with pytest.raises(RuntimeError, match="engine step failed"):
        list(handle)
    assert handle.finish_reason == "error"
    e.runner.fail_at = None
    assert len(list(e.submit([4, 5], GREEDY))) == 10  # the thread is still serving
    e.shutdown()
    assert e.stats()["kv_blocks_used"] == 0


def test_requests_without_a_seed_get_distinct_streams_and_seeded_ones_keep_theirs():
    e = Engine(CountingRunner(), Scheduler(EngineConfig(block_size=4, num_blocks=64, max_model_len=64)), seed=1)
    e.submit([1], SamplingParams())
    e.submit([1], SamplingParams())
    e.submit([1], SamplingParams(seed=42))
    e._read_mail(wait=False)
    a, b, c = e.scheduler.waiting
    assert a.noise_seed != b.noise_seed and c.noise_seed == 42


class _LazyStep:
    """A step of `AheadRunner` on its way: what it gives is worked out when it is read, from the
    tokens that the sequences hold by then (a step sent ahead is read after the step before it)."""

    device_tokens = None

    def __init__(self, out, ahead):
        self.out, self.ahead = out, ahead

    def results(self):
        if self.ahead:
            return [StepResult([sum(s.token_ids) % 97], s.num_tokens) for s in self.out.seqs]
        return [StepResult([sum(s.token_ids) % 97] if s.reaches_end(n) else [], s.num_computed_tokens + n)
                for s, n in zip(self.out.seqs, self.out.num_new_tokens)]  # fmt: skip


class AheadRunner(CountingRunner):
    """The same tokens as `CountingRunner` through the interface of a runner that can send a decode
    step to the GPU before the one before it was read."""

    def __init__(self):
        super().__init__()
        self.sent_ahead = 0

    def can_run_ahead(self, seqs):
        return True

    def launch(self, out, after=None):
        self.calls += 1
        if self.fail_at is not None and self.calls >= self.fail_at:
            raise RuntimeError("device fell over")
        self.sent_ahead += after is not None
        if after is not None:  # what the engine promises for such a step
            assert all(s.cache.tables[0] and len(s.cache.tables[0]) * 4 > s.num_tokens for s in out.seqs)
            assert out.num_new_tokens == [1] * len(out.seqs)
        return _LazyStep(out, after is not None)


@pytest.mark.parametrize("eos", [frozenset(), frozenset({7, 23, 61})])
def test_steps_sent_ahead_change_nothing_but_the_time(eos):
    """With and without steps sent ahead: the same tokens and finish reasons, for requests that end on
    a token, by length, at the longest sequence and by an abort in the middle; pages all given back."""
    params = [SamplingParams(temperature=0.0, max_tokens=m, ignore_eos=False) for m in (10, 3, 25, 1, 17)]

    def run(runner, **kw):
        cfg = EngineConfig(**{"block_size": 4, "num_blocks": 64, "max_model_len": 24, **kw})
        e = Engine(runner, Scheduler(cfg, eos))
        handles = [e.submit(p, q) for p, q in zip(PROMPTS, params)]
        steps = 0
        while e.step():
            steps += 1
            if steps == 6:
                e.abort(handles[2].id)
                late = e.submit([3, 1, 4, 1, 5], params[0])  # arrives while others decode
        handles.append(late)
        outs = [(list(h), h.finish_reason) for h in handles]
        assert e.stats()["kv_blocks_used"] == 0 and e.steps_in_flight == 0
        return outs

    plain = run(CountingRunner())
    ahead_runner = AheadRunner()
    assert run(ahead_runner) == plain
    assert ahead_runner.sent_ahead >= 5
    reasons = {reason for _, reason in plain}
    assert {"length", "abort"} <= reasons and (not eos or "stop" in reasons)
    # a pool so small that requests are preempted: steps go ahead only while nobody has to make room
    tight = dict(num_blocks=10, max_num_seqs=3)
    assert run(AheadRunner(), **tight) == run(CountingRunner(), **tight)
    # every place taken and a queue behind: the queue cannot move, so steps still go ahead
    # (a request that ends on a token leaves its place one step later then, so the abort at the sixth
    # step finds its request a token further or less: that one is compared up to the shorter reply)
    full = AheadRunner()
    ahead, waited = run(full, max_num_seqs=2), run(CountingRunner(), max_num_seqs=2)
    assert full.sent_ahead >= 5
    assert ahead[:2] + ahead[3:] == waited[:2] + waited[3:]
    (a, reason_a), (w, reason_w) = ahead[2], waited[2]
    n = min(len(a), len(w))
    assert a[:n] == w[:n] and reason_a == reason_w == "abort"


def test_a_failing_step_leaves_no_step_behind_it():
    """The launch of a step sent ahead fails: the requests fail, nothing stays on its way, and the
    engine serves the next request as if nothing had happened."""
    e = Engine(AheadRunner(), Scheduler(EngineConfig(block_size=4, num_blocks=64, max_model_len=64), frozenset()))
    e.runner.fail_at = 4  # the prompt, a decode step, one sent ahead, then the failure
    e.start()
    handle = e.submit([1, 2, 3], GREEDY)
    with pytest.raises(RuntimeError, match="engine step failed"):
        list(handle)
    e.runner.fail_at = None
    alone = engine().generate([[4, 5]], GREEDY)[0]
    assert list(e.submit([4, 5], GREEDY)) == alone
    e.shutdown()
    assert e.steps_in_flight == 0 and e.stats()["kv_blocks_used"] == 0 and e.runner.sent_ahead > 2

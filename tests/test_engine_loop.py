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
    e._drain_inbox(block=False)
    a, b, c = e.scheduler.waiting
    assert a.noise_seed != b.noise_seed and c.noise_seed == 42

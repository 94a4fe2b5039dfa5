"""The two tiny workloads as they are stated for this engine, run through the whole stack (engine,
scheduler, cache, step function, kernels, sampler) in 32-bit:

  A: prompts of 5, 17 and 33 token ids, pages of 16, 16 tokens decoded greedily;
  B: prompts of 1, 9, 40 and 71 token ids, pages of 8, a budget of 24 tokens a step, 20 tokens
     decoded, once greedily and once with temperature 0.7 under fixed seeds.

Weights: matrices N(0, 0.02), gains 1 + N(0, 0.1) (the `tiny` fixture).  For each workload the replies
are the same however the scheduler cuts the work: all requests together, each alone, prompts in portions
under the budget of 24 beside decoded tokens, a pool so small that requests are evicted and recomputed,
and a second pass that finds its prompts in the prefix cache (the invariants of reference
tests/test_engine.py:21-49).  Greedy replies are the plain model's; every sampled token has mass in the
distribution that the plain sampler forms from the plain model's logits at its place, and a seeded
request's stream does not depend on who shares its batches (reference tests/test_sampler.py:50-61, here
as a property of the engine)."""

import pytest
import torch

from tests import plain_qwen3 as plain
from tests import replay_cases as rc
from tests.conftest import write_model_dir

pytestmark = pytest.mark.gpu

WORKLOADS = {
    "A": {"prompts": (5, 17, 33), "page": 16, "decoded": 16},
    "B": {"prompts": (1, 9, 40, 71), "page": 8, "decoded": 20},
}
BUDGET = 24


@pytest.fixture(scope="module")
def served(tiny, tmp_path_factory):
    from atomserve_amd.weights import load_model

    name, raw, weights = tiny
    path = write_model_dir(str(tmp_path_factory.mktemp(f"workload{name}")), raw, weights, torch.float32)
    model, _, _ = load_model(path, torch.float32, "cuda:0")
    work = WORKLOADS[name]
    prompts = [rc.random_ids(raw["vocab_size"], n, seed=3000 + n) for n in work["prompts"]]
    return raw, weights, model, work, prompts


def every_cut(model, work, prompts, params):
    """The replies of the same requests under five ways of scheduling them, by name."""
    from atomserve_amd.config import EngineConfig
    from atomserve_amd.engine.engine import create_engine

    page, longest = work["page"], max(map(len, prompts)) + work["decoded"]
    limit = -(-(longest + 1) // page) * page

    def engine(**kw):
        cfg = {"block_size": page, "num_blocks": 64, "max_model_len": limit, "max_num_seqs": 8, **kw}
        return create_engine(model, EngineConfig(**cfg))

    def run(eng, which=None):
        chosen = list(range(len(prompts))) if which is None else which
        handles = [eng.submit(prompts[i], params[i]) for i in chosen]
        while eng.step():
            pass
        got = [list(h) for h in handles]  # reading a handle to its end also tells why it ended
        assert eng.stats()["kv_blocks_used"] == 0 and all(h.finish_reason == "length" for h in handles)
        return got

    replies = {"together": run(engine())}
    replies["alone"] = [run(engine(), [i])[0] for i in range(len(prompts))]
    chunked = engine(max_num_batched_tokens=BUDGET)
    replies["budget"] = run(chunked)
    assert chunked.stats()["steps"] > work["decoded"] + 1  # the prompts did come in portions
    # exactly the pages the prompts need, and at least what the longest request needs alone: every
    # request that grows takes the pages of a newer one, which is recomputed later
    tight = engine(num_blocks=max(sum(-(-len(p) // page) for p in prompts), limit // page))
    replies["evicted"] = run(tight)
    assert tight.stats()["preemptions"] > 0
    warm = engine()
    run(warm)
    before = warm.stats()["cached_prompt_tokens"]
    replies["cached"] = run(warm)
    assert warm.stats()["cached_prompt_tokens"] >= before + (max(map(len, prompts)) // page) * page
    replies["uncached"] = run(engine(enable_prefix_caching=False))
    return replies


def test_greedy_replies_are_the_plain_models_under_every_cut(served):
    from atomserve_amd.engine.sequence import SamplingParams

    raw, weights, model, work, prompts = served
    params = [SamplingParams(temperature=0.0, max_tokens=work["decoded"], ignore_eos=True)] * len(prompts)
    replies = every_cut(model, work, prompts, params)
    want = [plain.greedy(raw, weights, p, work["decoded"]) for p in prompts]
    for cut, got in replies.items():
        assert got == want, cut


def test_seeded_replies_are_the_same_under_every_cut_and_lie_in_the_plain_distribution(served):
    from atomserve_amd.engine.sequence import SamplingParams

    raw, weights, model, work, prompts = served
    params = [SamplingParams(temperature=0.7, max_tokens=work["decoded"], ignore_eos=True, seed=40 + i)
              for i in range(len(prompts))]  # fmt: skip
    replies = every_cut(model, work, prompts, params)
    first = replies["together"]
    for cut, got in replies.items():
        assert got == first, cut
    assert all(len(reply) == work["decoded"] for reply in first)
    assert any(len(set(reply)) > 3 for reply in first)  # draws, not one token again and again
    # another seed is another stream; the same seed beside other neighbours is the same stream (above)
    greedy = [plain.greedy(raw, weights, p, work["decoded"]) for p in prompts]
    assert first != greedy
    for p, q, reply in zip(prompts, params, first):
        ref = plain.logits(raw, weights, p + reply)[len(p) - 1 : -1]
        for place, token in enumerate(reply):
            dist = plain.sampling_distribution(ref[place], q.temperature, q.top_k, q.top_p)
            assert dist[token] > 0, f"token {token} at place {place} has no mass in the plain distribution"

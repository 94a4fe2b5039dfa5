"""The sampler as the engine calls it (sequences with their own settings), on hand-made logits;
each test pins one rule of the pipeline (cases of reference tests/test_sampler.py:28-83)."""

import pytest
import torch

from atomserve_amd.engine.sequence import SamplingParams, Sequence

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
PROBS = torch.tensor([0.4, 0.3, 0.2, 0.1])


@pytest.fixture(scope="module")
def sampler():
    from atomserve_amd.sampling import Sampler

    return Sampler(DEV)


def seqs(n, output_ids=None, **params):
    tokens = [0, *(output_ids or [])]
    out = [Sequence(i, list(tokens), SamplingParams(**params), num_prompt_tokens=1) for i in range(n)]
    for i, s in enumerate(out):
        if s.params.seed is None:
            s.noise_seed = 1000 + 7919 * i  # what the engine does at submit for requests without a seed
    return out


def draws(sampler, n, **params):
    logits = PROBS.log().repeat(n, 1).to(DEV)
    return torch.tensor(sampler.sample(logits, seqs(n, **params)))


def test_temperature_zero_is_argmax(sampler):
    logits = torch.tensor([[0.1, 3.0, 0.2], [5.0, 1.0, 0.0]], device=DEV)
    assert sampler.sample(logits, seqs(2, temperature=0.0)) == [1, 0]
    assert sampler.sample(torch.empty(0, 10, device=DEV), []) == []


def test_draws_follow_the_distribution_and_the_truncations(sampler):
    counts = draws(sampler, 20000, temperature=1.0, top_k=0, top_p=1.0).bincount(minlength=4)
    assert torch.allclose(counts / 20000, PROBS, atol=0.015)
    assert set(draws(sampler, 2000, temperature=1.0, top_k=2, top_p=1.0).tolist()) == {0, 1}
    assert set(draws(sampler, 200, temperature=1.0, top_k=1, top_p=1.0).tolist()) == {0}
    assert set(draws(sampler, 2000, temperature=1.0, top_k=0, top_p=0.6).tolist()) == {0, 1}
    assert set(draws(sampler, 200, temperature=1.0, top_k=0, top_p=0.01).tolist()) == {0}


def test_seeded_requests_repeat_regardless_of_batch_neighbours(sampler):
    torch.manual_seed(0)
    logits = torch.randn(1, 1000, device=DEV)
    other = seqs(2, temperature=0.8, top_k=500, top_p=0.9)
    other[0].id, other[1].id = 10, 11
    a, b = [], []
    seeded = seqs(1, temperature=1.0, top_k=50, top_p=1.0, seed=7)[0]
    for _ in range(20):
        a.append(sampler.sample(logits, [seeded])[0])
        seeded.token_ids.append(a[-1])
    seeded = seqs(1, temperature=1.0, top_k=50, top_p=1.0, seed=7)[0]
    for _ in range(20):
        b.append(sampler.sample(logits.repeat(3, 1), [other[0], seeded, other[1]])[1])
        seeded.token_ids.append(b[-1])
    assert a == b and len(set(a)) > 1


def test_presence_penalty_discourages_generated_tokens(sampler):
    logits = torch.tensor([[2.0, 1.9, 0.0]], device=DEV)
    assert sampler.sample(logits, seqs(1, output_ids=[0], temperature=0.0)) == [0]
    assert sampler.sample(logits, seqs(1, output_ids=[0], temperature=0.0, presence_penalty=0.5)) == [1]
    assert torch.equal(logits, torch.tensor([[2.0, 1.9, 0.0]], device=DEV))  # the caller's logits are untouched


@pytest.mark.parametrize("seed", [None, 3])
def test_greedy_and_sampled_rows_mix_in_one_batch(sampler, seed):
    logits = torch.tensor([[0.0, 9.0, 0.0], [0.0, 0.0, 9.0]], device=DEV)
    batch = seqs(1, temperature=0.0) + seqs(1, temperature=1.0, top_k=1, seed=seed)
    batch[1].id = 1
    assert sampler.sample(logits, batch) == [1, 2]


def test_top_k_beyond_what_is_ranked_keeps_the_k_largest(sampler):
    """A top-k of thousands is a floor on the logit (the k-th largest, found over the whole row):
    draws come from those k tokens only, with the plain distribution's frequencies, also with a
    top-p on top."""
    from tests import plain_qwen3 as plain

    torch.manual_seed(3)
    V, k, n = 6000, 2500, 3000
    row = torch.randn(V) * 0.7
    row[torch.randperm(V)[:5]] += 3.0  # a few likely tokens, so that frequencies can be compared
    logits = row.repeat(n, 1).to(DEV)
    for top_p in (1.0, 0.9):
        batch = seqs(n, temperature=1.0, top_k=k, top_p=top_p)
        got = torch.tensor(sampler.sample(logits, batch))
        dist = plain.sampling_distribution(row, 1.0, k, top_p)
        assert bool((dist[got] > 0).all()), "a token outside the k largest (or the top-p set) was drawn"
        dist = dist / dist.sum()
        top = dist.topk(5).indices
        freq = torch.bincount(got, minlength=V)[top].double() / n
        sigma = (dist[top] * (1 - dist[top]) / n).sqrt()
        assert bool(((freq - dist[top]).abs() <= 5 * sigma).all()), (freq, dist[top])
    # the k-th largest has equals: they all stay (k = 1100 reaches into a run of equal logits)
    tied = torch.full((V,), -2.0)
    tied[:1000] = torch.linspace(3.0, 1.0, 1000)
    tied[1000:1400] = 0.5  # 400 equal logits across the k-th place
    got = set(sampler.sample(tied.repeat(4000, 1).to(DEV), seqs(4000, temperature=2.0, top_k=1100, top_p=1.0)))
    assert max(got) < 1400 and len([t for t in got if t >= 1100]) > 0

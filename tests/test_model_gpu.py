"""The engine against the plain implementation on a real GPU, in 32-bit and in bfloat16:
the same requests whole, decoded one by one, in portions, and mixed with few pages."""

import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from tests import plain_qwen3 as plain
from tests import replay_cases as rc
from tests.conftest import ROOT, TINY, plain_random_weights, write_model_dir

pytestmark = pytest.mark.gpu

# fp32: the engine and the float64 plain implementation differ by fp32 rounding only (a multiple of the
# largest logit).  bf16: the bound is calibrated, trace by trace: what rounding the plain model's own
# activations to bfloat16 does to the same rows (tests/replay_cases.py `within_bounds`).
LENGTHS = {"A": 200, "B": 420}
PAGE = {"A": 16, "B": 8}  # each tiny configuration at its own page size


@pytest.fixture(scope="module", params=["A", "B"])
def setup(request, tmp_path_factory):
    name = request.param
    raw = TINY[name]
    weights = plain_random_weights(raw, seed=41 if name == "A" else 43, std=0.2, gain_std=0.2)
    path = write_model_dir(str(tmp_path_factory.mktemp(f"tiny{name}")), raw, weights, torch.bfloat16)
    return name, raw, weights, path, {}


def make_replay(path, dtype, max_tokens, block_size=16, max_live=4):
    from atomserve_amd.engine.replay import Replay

    return Replay(path, dtype, max_tokens, block_size=block_size, max_live=max_live)


def compare(replay, steps, requests, raw, weights, cache, dtype, **how):
    """Replays the trace against the plain model and holds the result to the bound of its precision."""
    result = rc.run_and_compare(replay, steps, requests, raw, weights, cache, noise=dtype == "bfloat16", **how)
    rc.within_bounds(result, dtype)
    return result


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_decoded_and_in_portions(setup, dtype):
    name, raw, weights, path, cache = setup
    ids = rc.random_ids(raw["vocab_size"], LENGTHS[name], seed=1)
    requests = {"a": ids}
    for steps in (rc.whole("a", ids), rc.prefill_then_decode("a", ids), rc.portions("a", ids)):
        replay = make_replay(path, dtype, rc.live_token_bound(steps), PAGE[name])
        assert compare(replay, steps, requests, raw, weights, cache, dtype).rows >= 33
        assert replay.manager.num_free == replay.manager.num_blocks  # everything was given back


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mixed_requests_with_pages_used_again(setup, dtype):
    name, raw, weights, path, cache = setup
    lengths = [70, 33, 150, 64, 97, 20, 129, 65] if name == "A" else [90, 300, 64, 17, 257, 128, 40, 200]
    requests = {f"r{i}": rc.random_ids(raw["vocab_size"], n, seed=100 + i) for i, n in enumerate(lengths)}
    steps = rc.mixed(requests, seed=5)
    bound = rc.live_token_bound(steps)
    assert bound < sum(-(-n // 64) * 64 for n in lengths)  # fewer pages than all requests need: reuse
    replay = make_replay(path, dtype, bound, PAGE[name])
    assert compare(replay, steps, requests, raw, weights, cache, dtype).rows > 200
    assert replay.manager.num_free == replay.manager.num_blocks


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("block_size", [8, 16, 32, 48])
def test_every_cut_at_other_page_sizes(setup, dtype, block_size):
    """Whole, decoded, in portions and mixed with pages used again, at pages of 8, 16, 32 and 48
    tokens (48 divides neither the 64 queries of a tile nor the 64 tokens that the pool is counted
    in; 8 sends bfloat16 through the general attention kernel): the same logits."""
    name, raw, weights, path, cache = setup
    lengths = [70, 33, 150, 64, 97, 20] if name == "A" else [90, 300, 64, 17, 257, 128]
    requests = {f"r{i}": rc.random_ids(raw["vocab_size"], n, seed=100 + i) for i, n in enumerate(lengths)}
    first = ("r2", requests["r2"])
    mixed = rc.mixed(requests, seed=block_size)
    assert rc.live_token_bound(mixed) < sum(-(-n // 64) * 64 for n in lengths)
    for steps in (rc.whole(*first), rc.prefill_then_decode(*first), rc.portions(*first), mixed):
        replay = make_replay(path, dtype, rc.live_token_bound(steps), block_size)
        assert compare(replay, steps, requests, raw, weights, cache, dtype).rows >= 33
        assert replay.manager.num_free == replay.manager.num_blocks


@pytest.mark.parametrize("seed", range(6))
def test_random_traces_in_32_bit(setup, seed):
    """Requests, portion sizes around the edges of pages and tiles, how many are live and how much
    of each is prompt drawn at random, the pool as small as the trace allows: in 32-bit every
    wanted row is the plain model's to a tenth of the bound, so anything a cut or a reused page
    breaks shows far above rounding."""
    import random

    name, raw, weights, path, _ = setup
    rng = random.Random(7 * seed + (name == "B"))
    longest = min(raw["max_position_embeddings"], rng.choice([40, 130, 250]))
    requests = {f"r{i}": rc.random_ids(raw["vocab_size"], rng.randint(2, longest), seed=900 + 10 * seed + i)
                for i in range(rng.randint(2, 7))}  # fmt: skip
    sizes = tuple(rng.choice([2, 3, 5, 8, 9, 15, 16, 17, 31, 32, 33, 63, 64, 65, 100]) for _ in range(6))
    steps = rc.mixed(requests, seed=seed, max_live=rng.randint(1, 4), prompt_fraction=rng.choice([0.3, 0.6, 0.95]), sizes=sizes)
    replay = make_replay(path, "float32", rc.live_token_bound(steps), rng.choice([4, 8, 16, 24, 64]))
    worst, scale, rows = rc.run_and_compare(replay, steps, requests, raw, weights, {})
    assert rows > 0 and worst <= 0.3 * rc.TOL_FLOAT32 * max(scale, 1.0)
    assert replay.manager.num_free == replay.manager.num_blocks


@pytest.mark.parametrize("seed", range(16))
def test_configurations_drawn_at_random(seed, tmp_path):
    """Every size and option of the configuration drawn anew (head widths in steps of 16 up to 256,
    groups that are no power of two, one kv head, widths from 24 to 520, an odd vocabulary, one to
    four layers, eps, theta, tied or not): whole, decoded, in portions and mixed, in both precisions.
    The matrices shrink with the width so that scores and logits stay of order one to ten."""
    import random

    rng = random.Random(seed)
    kv, group, h = rng.choice([1, 2, 3, 4, 5]), rng.choice([1, 2, 3, 4, 5, 6, 7, 8]), rng.choice([24, 40, 56, 72, 88, 104, 136, 200, 264, 520])
    raw = dict(TINY["A"], vocab_size=rng.choice([50, 97, 1031, 5003]), hidden_size=h,
               intermediate_size=rng.choice([32, 48, 72, 100, 264, 2 * rng.randint(8, 300)]),
               num_hidden_layers=rng.randint(1, 4), num_attention_heads=kv * group, num_key_value_heads=kv,
               head_dim=16 * rng.randint(1, 16), rms_norm_eps=rng.choice([1e-6, 1e-5, 1e-3]),
               rope_theta=rng.choice([1e4, 5e5, 1e6]), tie_word_embeddings=rng.random() < 0.5,
               max_position_embeddings=512)  # fmt: skip
    weights = plain_random_weights(raw, seed=seed + 7, std=min(0.2, 1.0 / h**0.5), gain_std=0.2)
    path = write_model_dir(str(tmp_path / "drawn"), raw, weights, torch.bfloat16)
    requests = {f"r{i}": rc.random_ids(raw["vocab_size"], rng.randint(34, 150), seed=seed * 10 + i) for i in range(4)}
    first = next(iter(requests.items()))
    cases = [rc.whole(*first), rc.prefill_then_decode(*first), rc.portions(*first), rc.mixed(requests, seed=seed)]
    cache = {}
    page = rng.choice([8, 16, 32, 48, 64])
    for dtype in ("float32", "bfloat16"):
        for steps in cases:
            replay = make_replay(path, dtype, rc.live_token_bound(steps), page)
            assert compare(replay, steps, requests, raw, weights, cache, dtype).rows > 0
            assert replay.manager.num_free == replay.manager.num_blocks


def test_the_error_of_bfloat16_is_what_rounding_alone_does(setup):
    """The bound of the bfloat16 tests above is a few rounding steps of the largest logit.  This one
    is calibrated: the plain model with its activations rounded to bfloat16 at the places where an
    engine that stores them so must round (tests/plain_qwen3.py `storage`) moves away from the exact
    logits by some root mean square; the engine, whole prompts and decoded tokens alike, is no
    further from the exact logits than one and a half times that, over all logits of a request."""
    name, raw, weights, path, cache = setup
    ids = rc.random_ids(raw["vocab_size"], LENGTHS[name], seed=1)
    exact = plain.logits(raw, weights, ids, batched=True).float()
    rounded = plain.logits(raw, weights, ids, batched=True, storage=torch.bfloat16).float()
    noise = float((rounded - exact).pow(2).mean().sqrt())
    for steps in (rc.whole("a", ids), rc.prefill_then_decode("a", ids, tail=64), rc.portions("a", ids)):
        replay = make_replay(path, "bfloat16", rc.live_token_bound(steps), PAGE[name])
        at, sq, n = 0, 0.0, 0
        for s in steps:
            logits = replay.step(s["entries"], s["end"])
            e = s["entries"][0]
            for k, w in enumerate(e["want"]):
                sq += float((logits[k] - exact[at + w]).pow(2).sum())
                n += exact.shape[1]
            at += len(e["tokens"])
        assert n and (sq / n) ** 0.5 <= 1.5 * noise, f"engine {(sq / n) ** 0.5:.3e} against rounding {noise:.3e}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens_and_long_decoding(setup, dtype):
    name, raw, weights, path, cache = setup
    n = LENGTHS[name]
    ids = rc.random_ids(raw["vocab_size"], n, seed=2)
    steps = [{"step": i, "entries": [{"id": "d", "tokens": [ids[i]], "want": [0]}], "end": []} for i in range(n)]
    replay = make_replay(path, dtype, n + 64, PAGE[name])
    assert compare(replay, steps, {"d": ids}, raw, weights, cache, dtype).rows == n


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decoding_across_the_context_bound_of_a_captured_graph(dtype, tmp_path):
    """Replayed decode steps are captured for contexts up to a multiple of 1,024 tokens; a request
    that decodes from 1,009 to 1,040 tokens passes from one captured step to the next."""
    raw = dict(TINY["A"], max_position_embeddings=2048)
    weights = plain_random_weights(raw, seed=47, std=0.2, gain_std=0.2)
    path = write_model_dir(str(tmp_path / "long"), raw, weights, torch.bfloat16)
    ids = rc.random_ids(raw["vocab_size"], 1040, seed=6)
    steps = rc.prefill_then_decode("a", ids)
    replay = make_replay(path, dtype, rc.live_token_bound(steps))
    assert compare(replay, steps, {"a": ids}, raw, weights, {}, dtype).rows == 33
    assert len(replay.runner.decode_graphs.graphs) == 2


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("num_requests", [3, 13, 21, 40, 100])
def test_decode_graphs_replay_what_eager_steps_give(setup, dtype, num_requests):
    """Decode steps replayed as captured graphs against the same steps launched kernel by kernel:
    the same logits at every step, over several replays with eager work (a new request's prompt)
    and synchronisations between them, for row counts in the small buckets (one and two row tiles
    of this package's products) and the large ones (whose matrix products are the library's).  The
    last step's logits are also the plain model's."""
    from atomserve_amd.weights.loader import load_model

    name, raw, weights, path, cache = setup
    model, _, _ = load_model(path, getattr(torch, dtype), "cuda:0")
    graphs_against_eager(model, raw, weights, dtype, num_requests, torch.float64)


def graphs_against_eager(model, raw, weights, dtype, num_requests, plain_dtype):
    from atomserve_amd.cache.manager import CacheManager
    from atomserve_amd.engine.batch import Row
    from atomserve_amd.engine.runner import ModelRunner

    vocab = raw["vocab_size"]
    prompts = [rc.random_ids(vocab, 5 + 3 * (i % 11), seed=300 + i) for i in range(num_requests)]
    later = [rc.random_ids(vocab, 12, seed=400 + i) for i in range(num_requests)]  # the tokens decoded, given
    extra = rc.random_ids(vocab, 40, seed=500)
    seen = {}
    for use_graphs in (True, False):
        manager = CacheManager(model.cache_requests(), 16, 8 * num_requests + 16, num_requests + 2)
        runner = ModelRunner(model, manager, use_graphs=use_graphs)
        live = [[manager.new_request(), 0] for _ in range(num_requests)]

        def rows_of(token_lists, who=live):
            rows = []
            for state, tokens in zip(who, token_lists):
                assert manager.reserve(state[0], state[1], len(tokens))
                rows.append(Row(list(tokens), state[1], state[0].tables, [len(tokens) - 1], state[0].state_slot))
                state[1] += len(tokens)
            return rows

        out = [runner.step(rows_of(prompts)).float().cpu()]
        for step in range(8):
            if step == 3:  # eager work between the replays: another request's prompt, alone in its step
                other = [[manager.new_request(), 0]]
                out.append(runner.step(rows_of([extra], other)).float().cpu())
                torch.cuda.synchronize()
            out.append(runner.step(rows_of([[t[step]] for t in later])).float().cpu())
        if use_graphs and dtype in ("float32", "bfloat16"):
            assert runner.decode_graphs.graphs, "no step was replayed from a graph"
        seen[use_graphs] = out
    # the plain model at the last step's rows of three requests: exact, and what rounding its activations
    # to bfloat16 does to it there (the measure of every bfloat16 bound below)
    against_plain = {use_graphs: rc.Comparison() for use_graphs in seen}
    for i in (0, num_requests // 2, num_requests - 1):
        ids = prompts[i] + later[i][:8]
        ref = plain.logits(raw, weights, ids, dtype=plain_dtype, batched=True)[-1].float()
        rounded = plain.logits(raw, weights, ids, dtype=plain_dtype, batched=True, storage=torch.bfloat16)[-1].float()
        for use_graphs, out in seen.items():
            result = against_plain[use_graphs]
            result.err.add(out[-1][i] - ref)
            result.noise.add(rounded - ref)
            result.scale = max(result.scale, float(ref.abs().max()))
    for result in against_plain.values():
        rc.within_bounds(result, dtype)
    # a replayed step is padded to its bucket and cuts contexts by the bucket's bound, so sums are
    # taken in another order: the same numbers up to rounding, which is twice over what either is from
    # the exact logits
    noise = against_plain[True].noise
    apart = rc.Spread()
    for a, b in zip(seen[True], seen[False]):
        assert a.shape == b.shape and torch.isfinite(a).all()
        apart.add(a - b)
    if dtype == "float32":
        assert apart.worst <= rc.TOL_FLOAT32 * max(against_plain[True].scale, 1.0)
    else:
        assert apart.rms <= 2 * rc.BF16_RMS_FACTOR * noise.rms and apart.worst <= 2 * rc.BF16_WORST_FACTOR * noise.worst, (
            f"replayed - eager: rms {apart.rms:.3e} max {apart.worst:.3e}; rounding alone: rms {noise.rms:.3e} max {noise.worst:.3e}")  # fmt: skip


def test_captured_steps_are_dropped_and_captured_again(setup):
    """Only so many captured steps are kept.  Three groups of requests (one, three and six rows:
    three buckets) decode in turn with room for two captured steps, so every step finds its own
    dropped, captures it again from the shared memory pool and replays it: the logits are those of
    eager steps throughout."""
    from atomserve_amd.cache.manager import CacheManager
    from atomserve_amd.engine.batch import Row
    from atomserve_amd.engine.runner import ModelRunner
    from atomserve_amd.weights.loader import load_model

    name, raw, weights, path, _ = setup
    model, _, _ = load_model(path, torch.float32, "cuda:0")
    vocab = raw["vocab_size"]
    groups = [[rc.random_ids(vocab, 7 + 5 * i + j, seed=600 + 10 * i + j) for j in range(n)] for i, n in enumerate((1, 3, 6))]
    seen = {}
    for use_graphs in (True, False):
        manager = CacheManager(model.cache_requests(), 16, 64, 16)
        runner = ModelRunner(model, manager, use_graphs=use_graphs)
        if use_graphs:
            runner.decode_graphs.MAX_GRAPHS = 2
        out = []
        live = [[[manager.new_request(), 0] for _ in group] for group in groups]
        for turn in range(5):
            for group, states in zip(groups, live):
                rows = []
                for ids, state in zip(group, states):
                    tokens = ids[:-4] if turn == 0 else [ids[len(ids) - 5 + turn]]
                    assert manager.reserve(state[0], state[1], len(tokens))
                    rows.append(Row(tokens, state[1], state[0].tables, [len(tokens) - 1], -1))
                    state[1] += len(tokens)
                out.append(runner.step(rows).float().cpu())
                if use_graphs:
                    assert len(runner.decode_graphs.graphs) <= 2
        seen[use_graphs] = out
    ref = plain.logits(raw, weights, groups[2][5])[-1].float()
    bound = rc.TOL_FLOAT32 * max(1.0, float(ref.abs().max()))
    for a, b in zip(seen[True], seen[False]):
        assert float((a - b).abs().max()) <= bound
    assert float((seen[True][-1][5] - ref).abs().max()) <= bound


@pytest.fixture(scope="module")
def like_8b(tmp_path_factory):
    raw = {**TINY_B_LIKE_8B}
    weights = plain_random_weights(raw, seed=78, std=0.02, gain_std=0.1)
    return raw, weights, write_model_dir(str(tmp_path_factory.mktemp("real_graphs")), raw, weights, torch.bfloat16)


@pytest.mark.parametrize("dtype,counts", [("bfloat16", (3, 9, 13, 16, 21, 40)), ("float32", (9, 16))])
def test_decode_graphs_at_real_layer_sizes(like_8b, dtype, counts):
    """The same at Qwen3-8B's layer sizes, where the row count of a decode step chooses its matrix products:
    up to 8 rows the few-rows kernels with the residual sum and the norm folded in, 9 to 16 rows the tile
    products with one row tile (split sums into the norm, the gated tile), 17 to 64 rows those with more
    row tiles or the library's with the candidate that the warm-up's trials chose.  Replays of the captured
    steps give what eager steps give, replay after replay, and what the plain model gives."""
    from atomserve_amd.weights.loader import load_model

    raw, weights, path = like_8b
    model, _, _ = load_model(path, getattr(torch, dtype), "cuda:0")
    for num_requests in counts:
        graphs_against_eager(model, raw, weights, dtype, num_requests, torch.float32)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(setup, dtype, tmp_path):
    """The program itself, as a user starts it: JSON lines in, <step>.f32 files and `done` lines out."""
    name, raw, weights, path, cache = setup
    ids = rc.random_ids(raw["vocab_size"], 50, seed=3)
    other = rc.random_ids(raw["vocab_size"], 21, seed=4)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": ids[:30], "want": [0, 29]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": ids[30:33], "want": []}, {"id": "c", "tokens": [], "want": []},
                                {"id": "b", "tokens": other, "want": [20]}], "end": ["b"]},  # fmt: skip
        {"step": 2, "entries": [{"id": "a", "tokens": ids[33:], "want": [16]}], "end": ["a"]},
        {"step": 3, "entries": [], "end": ["c"]},  # nothing to run, nothing to write
    ]
    out = tmp_path / "out"
    # the cache's geometry comes with the trace (a first line) or on the command line
    header = [{"geometry": {"block_size": 8, "pages": 16, "max_live": 3}}] if name == "B" else []
    geometry_flags = [] if name == "B" else ["--block-size", "32", "--max-live", "3"]
    proc = subprocess.run(
        [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", path, "--dtype", dtype, "--out", str(out),
         "--max-tokens", "128", *geometry_flags],
        input="\n".join(json.dumps(s) for s in header + steps) + "\n", capture_output=True, text=True, timeout=600,
    )  # fmt: skip
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert proc.stdout.split() == ["done", "0", "done", "1", "done", "2", "done", "3"]
    assert sorted(os.listdir(out)) == ["0.f32", "1.f32", "2.f32"]
    got0 = np.fromfile(out / "0.f32", dtype="<f4").reshape(2, -1)
    got1 = np.fromfile(out / "1.f32", dtype="<f4").reshape(1, -1)
    got2 = np.fromfile(out / "2.f32", dtype="<f4").reshape(1, -1)
    result, cache = rc.Comparison(), {}
    for got, rid, seq, place in ((got0[0], "a", ids, 0), (got0[1], "a", ids, 29), (got1[0], "b", other, 20), (got2[0], "a", ids, 49)):
        want = rc.plain_rows(raw, weights, seq, cache, rid, False)[place]
        result.err.add(torch.from_numpy(got.copy()) - want)
        result.noise.add(rc.plain_rows(raw, weights, seq, cache, rid, True)[place] - want)
        result.scale = max(result.scale, float(want.abs().max()))
    rc.within_bounds(result, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_greedy_generation_through_the_entry_point(setup, dtype):
    """Greedy tokens through engine, scheduler, cache and kernels equal recomputing the whole
    sequence for every token; batched, chunked and preempted runs give the same tokens (fp32)."""
    from atomserve_amd.config import EngineConfig
    from atomserve_amd.engine.engine import create_engine
    from atomserve_amd.engine.sequence import SamplingParams
    from atomserve_amd.weights import load_model

    name, raw, weights, path, _ = setup
    model, _, _ = load_model(path, dtype, "cuda:0")
    prompts = [rc.random_ids(raw["vocab_size"], n, seed=200 + n) for n in (5, 17, 33, 1)]
    params = SamplingParams(temperature=0.0, max_tokens=20, ignore_eos=True)
    bs = 16 if name == "A" else 8

    def engine(**kw):
        cfg = {"block_size": bs, "num_blocks": 64, "max_model_len": 128, "max_num_seqs": 8, **kw}
        return create_engine(model, EngineConfig(**cfg))

    together = engine().generate(prompts, params)
    if dtype == torch.float32:
        assert together == [plain.greedy(raw, weights, p, 20) for p in prompts]
        assert engine(max_num_batched_tokens=8, max_num_seqs=4).generate(prompts, params) == together
        # exactly the pages the prompts need: every request that grows evicts a newer one
        tight = engine(num_blocks=sum(-(-len(p) // bs) for p in prompts), max_model_len=64)
        assert tight.generate(prompts, params) == together
        assert tight.stats()["preemptions"] > 0 and tight.stats()["kv_blocks_used"] == 0
        # the same prompts again on one engine: their full pages are found in the prefix cache
        warm = engine()
        assert warm.generate(prompts, params) == together
        before = warm.stats()["cached_prompt_tokens"]
        assert warm.generate(prompts, params) == together
        assert warm.stats()["cached_prompt_tokens"] >= before + (33 // bs) * bs
        assert engine(enable_prefix_caching=False).generate(prompts, params) == together
    else:
        # bf16 may flip near-ties; every token must still be nearly the best under the plain logits: two
        # logits, each as far off as the engine may be (the bound of the replay tests, from what rounding
        # alone does to the plain model over this request)
        for p, out in zip(prompts, together):
            ref = plain.logits(raw, weights, p + out, batched=True)[len(p) - 1 : -1]
            rounded = plain.logits(raw, weights, p + out, batched=True, storage=torch.bfloat16)[len(p) - 1 : -1]
            slack = 2 * rc.BF16_WORST_FACTOR * float((rounded - ref).abs().max())
            for place, t in enumerate(out):
                assert ref[place, t] >= ref[place].max() - slack


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_decode_steps_sent_ahead_give_the_same_tokens(setup, dtype):
    """While the running requests only decode, the engine sends the next step to the GPU before it has
    read this one's tokens, and the GPU passes them on.  Seeded sampling, greedy rows, requests that
    stop on a token, at their length and at the longest sequence, a request that arrives in the middle
    and one that is aborted: token for token what the engine gives when it waits for every step."""
    from atomserve_amd.config import EngineConfig
    from atomserve_amd.engine.engine import create_engine
    from atomserve_amd.engine.sequence import SamplingParams
    from atomserve_amd.weights import load_model

    name, raw, weights, path, _ = setup
    model, _, _ = load_model(path, dtype, "cuda:0")
    vocab = raw["vocab_size"]
    prompts = [rc.random_ids(vocab, n, seed=700 + n) for n in (3, 18, 40, 9, 26)]
    params = [SamplingParams(temperature=0.8, top_k=12, top_p=0.9, max_tokens=30, seed=5),
              SamplingParams(temperature=0.0, max_tokens=7, ignore_eos=True),
              SamplingParams(temperature=1.0, top_k=0, top_p=1.0, max_tokens=60, seed=6),
              SamplingParams(temperature=0.6, top_k=20, top_p=0.95, max_tokens=60, seed=7, ignore_eos=True),
              SamplingParams(temperature=0.0, max_tokens=45)]  # fmt: skip
    eos = frozenset(range(0, vocab, 9))  # a ninth of the vocabulary ends a request: some stop early

    def run(run_ahead):
        cfg = EngineConfig(block_size=16, num_blocks=64, max_model_len=64, max_num_seqs=8, max_num_batched_tokens=64)
        engine = create_engine(model, cfg, eos)
        engine.run_ahead = run_ahead
        handles = [engine.submit(p, q) for p, q in zip(prompts, params)]
        steps, sent = 0, 0
        while engine.step():
            steps += 1
            sent += engine.steps_in_flight > 0
            if steps == 5:
                engine.abort(handles[3].id)
                handles.append(engine.submit(prompts[0][::-1] + prompts[1], params[0]))
        assert engine.stats()["kv_blocks_used"] == 0
        return [(list(h), h.finish_reason) for h in handles], sent

    waited, none_sent = run(False)
    ahead, sent = run(True)
    assert none_sent == 0 and sent >= 10
    assert ahead == waited
    assert {reason for _, reason in waited} >= {"stop", "length", "abort"}


def test_steps_sent_ahead_while_the_batch_shrinks_across_kernel_choices(setup):
    """Seventeen and thirty-three requests decode while some stop on a token: a request that has
    stopped rides one step too many, so the steps sent ahead cross from 17 rows to 16 and from 33 to
    32 (other row buckets, other matrix-product kernels) one step later than an engine that waits.
    In 32-bit every token is the same either way."""
    from atomserve_amd.config import EngineConfig
    from atomserve_amd.engine.engine import create_engine
    from atomserve_amd.engine.sequence import SamplingParams
    from atomserve_amd.weights import load_model

    name, raw, weights, path, _ = setup
    model, _, _ = load_model(path, torch.float32, "cuda:0")
    vocab = raw["vocab_size"]
    eos = frozenset(range(0, vocab, 23))
    for count in (17, 33):
        prompts = [rc.random_ids(vocab, 3 + (7 * i) % 20, seed=900 + i) for i in range(count)]
        params = [SamplingParams(temperature=0.8 if i % 3 else 0.0, top_k=15, max_tokens=20 + i % 5, seed=i, ignore_eos=i % 4 == 0)
                  for i in range(count)]  # fmt: skip
        results = []
        for run_ahead in (False, True):
            cfg = EngineConfig(block_size=16, num_blocks=160, max_model_len=64, max_num_seqs=40, max_num_batched_tokens=512)
            engine = create_engine(model, cfg, eos)
            engine.run_ahead = run_ahead
            handles = [engine.submit(p, q) for p, q in zip(prompts, params)]
            sizes = set()
            while engine.step():
                sizes.add(engine.counters["last_batch_seqs"])
            results.append([(list(h), h.finish_reason) for h in handles])
            assert engine.stats()["kv_blocks_used"] == 0
            assert count in sizes and min(sizes) < count - 1  # the batch did shrink across the boundary
        assert results[0] == results[1]
        assert {"stop", "length"} <= {reason for _, reason in results[0]}


def test_a_step_sent_ahead_may_be_the_first_of_its_graph(tmp_path):
    """Requests that decode from 1,015 and 1,020 tokens pass the context bound of the captured steps
    while steps are sent ahead: the step that is captured anew takes its tokens from the GPU like
    any other, and the tokens are those of an engine that waits for every step."""
    from atomserve_amd.config import EngineConfig
    from atomserve_amd.engine.engine import create_engine
    from atomserve_amd.engine.sequence import SamplingParams
    from atomserve_amd.weights import load_model

    raw = dict(TINY["A"], max_position_embeddings=2048)
    weights = plain_random_weights(raw, seed=47, std=0.2, gain_std=0.2)
    path = write_model_dir(str(tmp_path / "long"), raw, weights, torch.bfloat16)
    model, _, _ = load_model(path, torch.float32, "cuda:0")
    prompts = [rc.random_ids(raw["vocab_size"], n, seed=800 + n) for n in (1015, 1020)]
    params = SamplingParams(temperature=0.7, top_k=10, max_tokens=24, seed=3, ignore_eos=True)
    outs = []
    for run_ahead in (False, True):
        engine = create_engine(model, EngineConfig(block_size=16, num_blocks=160, max_model_len=1100, max_num_batched_tokens=2048))
        engine.run_ahead = run_ahead
        outs.append(engine.generate(prompts, params))
        assert len(engine.runner.decode_graphs.graphs) == 2 and engine.stats()["kv_blocks_used"] == 0
        # what the captured steps hold is reported: at least their logits, also when the allocator had room to spare
        logits_bytes = engine.runner.decode_graphs.most_rows * raw["vocab_size"] * 4
        assert engine.stats()["graph_bytes"] >= logits_bytes
    assert outs[0] == outs[1] and all(len(o) == 24 for o in outs[0])
    # a warm-up captures both context lengths that max_model_len allows ahead: the same tokens from graphs
    # that were captured on rows that only pad, and nothing is captured while the requests run
    engine = create_engine(model, EngineConfig(block_size=16, num_blocks=160, max_model_len=1100, max_num_seqs=3,
                                               max_num_batched_tokens=2048))  # fmt: skip
    assert engine.warm_up() == 6
    assert sorted(engine.runner.decode_graphs.graphs) == [(n, c) for n in (1, 2, 4) for c in (1024, 2048)]
    assert engine.generate(prompts, params) == outs[0] and len(engine.runner.decode_graphs.graphs) == 6


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_real_layer_sizes(dtype, tmp_path_factory):
    """Two layers of Qwen3-8B's sizes (hidden 4096, 32/8 heads of 128, intermediate 12288) with a
    smaller vocabulary: the kernels at the sizes they serve, whole, in portions and decoded."""
    raw = {**TINY_B_LIKE_8B}
    weights = plain_random_weights(raw, seed=77, std=0.02, gain_std=0.1)
    path = write_model_dir(str(tmp_path_factory.mktemp("real")), raw, weights, torch.bfloat16)
    ids = rc.random_ids(raw["vocab_size"], 150, seed=9)
    cache = {"a": plain.logits(raw, weights, ids, dtype=torch.float32).float()}
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": ids[:70], "want": list(range(0, 70, 7))}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": ids[70:75], "want": [0, 4]}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": ids[75:140], "want": [0, 64]}], "end": []}]  # fmt: skip
    steps += [{"step": 3 + i, "entries": [{"id": "a", "tokens": [ids[140 + i]], "want": [0]}], "end": []} for i in range(10)]
    replay = make_replay(path, dtype, 192)
    # the plain side runs in float32 here (the float64 copy of these weights would not be worth its memory)
    result = rc.run_and_compare(replay, steps, {"a": ids}, raw, weights, cache, plain_kwargs={"dtype": torch.float32},
                                noise=dtype == "bfloat16")  # fmt: skip
    assert result.rows == 24
    rc.within_bounds(result, dtype, tol32=1e-4)


TINY_B_LIKE_8B = {
    "architectures": ["Qwen3ForCausalLM"], "vocab_size": 20000, "hidden_size": 4096, "intermediate_size": 12288,
    "num_hidden_layers": 2, "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 128,
    "rms_norm_eps": 1e-6, "rope_theta": 1000000.0, "tie_word_embeddings": False, "max_position_embeddings": 4096,
    "hidden_act": "silu",
}  # fmt: skip


def test_a_folder_stored_in_32_bit_served_in_bfloat16(tmp_path):
    """Matrices follow the serving dtype; gains stored in 32-bit stay 32-bit and the kernels take
    them so."""
    raw = TINY["B"]
    weights = plain_random_weights(raw, seed=91, std=0.2, gain_std=0.2)
    path = write_model_dir(str(tmp_path / "m"), raw, weights, torch.float32)
    ids = rc.random_ids(raw["vocab_size"], 90, seed=6)
    replay = make_replay(path, "bfloat16", 128)
    assert replay.model.blocks[0].mixer.q_norm_weight.dtype == torch.float32
    assert replay.model.blocks[0].mixer.qkv_weight.dtype == torch.bfloat16
    steps = rc.portions("a", ids, sizes=(40, 3, 1, 1, 30, 15))
    assert compare(replay, steps, {"a": ids}, raw, weights, {}, "bfloat16").rows == 90


def test_command_line_generates(setup, capsys):
    """`atomserve <folder> --prompt-ids ...` end to end: greedy tokens equal the plain model's."""
    import json as js

    from atomserve_amd.engine.cli import main

    name, raw, weights, path, _ = setup
    prompts = [[3, 14, 15, 9, 2], [6, 5]]
    argv = [path, "--dtype", "fp32", "--temperature", "0", "--max-tokens", "5", "--ignore-eos", "--kv-mem-gb", "0.01",
            "--max-num-seqs", "4", "--max-batched-tokens", "16"]  # fmt: skip
    for p in prompts:
        argv += ["--prompt-ids", ",".join(map(str, p))]
    assert main(argv) == 0
    lines = [js.loads(line) for line in capsys.readouterr().out.splitlines() if line.startswith("{")]
    assert [r["output_ids"] for r in lines] == [plain.greedy(raw, weights, p, 5) for p in prompts]
    assert all(r["finish_reason"] == "length" for r in lines)
    # and with weights drawn from a seed instead of read from the folder
    assert main([path, "--random-weights", "3", "--temperature", "0.7", "--seed", "1", "--max-tokens", "4", "--prompt-ids", "1 2 3",
                 "--kv-mem-gb", "0.01", "--max-num-seqs", "4", "--max-batched-tokens", "16"]) == 0  # fmt: skip
    out = [js.loads(line) for line in capsys.readouterr().out.splitlines() if line.startswith("{")]
    assert len(out) == 1 and 1 <= len(out[0]["output_ids"]) <= 4
    assert all(0 <= t < raw["vocab_size"] for t in out[0]["output_ids"])
    # weights from a seed, greedy, 32-bit: the tokens are the plain model's on the same drawn weights
    from atomserve_amd.config.registry import architecture_for
    from atomserve_amd.weights.random_init import random_checkpoint

    arch = architecture_for(raw)
    drawn = random_checkpoint(arch, arch.parse_config(raw), 3, dtype=torch.float32, device="cuda:0")
    drawn = {k: v.cpu() for k, v in drawn.items()}
    assert main([path, "--random-weights", "3", "--dtype", "fp32", "--temperature", "0", "--max-tokens", "4", "--ignore-eos",
                 "--prompt-ids", "1 2 3", "--kv-mem-gb", "0.01", "--max-num-seqs", "4", "--max-batched-tokens", "16"]) == 0  # fmt: skip
    out = [js.loads(line) for line in capsys.readouterr().out.splitlines() if line.startswith("{")]
    assert out[0]["output_ids"] == plain.greedy(raw, drawn, [1, 2, 3], 4)
    # the same seed and settings twice: the same sampled tokens
    runs = []
    for _ in range(2):
        assert main([path, "--random-weights", "3", "--dtype", "fp32", "--temperature", "0.9", "--seed", "5", "--max-tokens", "6",
                     "--ignore-eos", "--prompt-ids", "4 5", "--kv-mem-gb", "0.01", "--max-num-seqs", "4",
                     "--max-batched-tokens", "16"]) == 0  # fmt: skip
        runs.append([js.loads(line) for line in capsys.readouterr().out.splitlines() if line.startswith("{")][0]["output_ids"])
    assert runs[0] == runs[1] and len(runs[0]) == 6


def test_command_line_says_what_a_folder_lacks(setup, tmp_path, capsys):
    """A folder that cannot be served ends the command with a line that says why, not with a traceback: a
    shard that the index names and the folder lacks (reference atomserve/loader.py:28-40), tensors of the
    wrong shape, a config.json of another architecture."""
    import json as js
    import shutil

    from atomserve_amd.engine.cli import main

    name, raw, weights, path, _ = setup
    tail = ["--prompt-ids", "1 2", "--kv-mem-gb", "0.01"]
    partial = str(tmp_path / "partial")
    shutil.copytree(path, partial)
    with open(os.path.join(partial, "model.safetensors.index.json"), "w") as f:
        js.dump({"weight_map": {k: ("model.safetensors" if i % 2 else "model-00002-of-00002.safetensors")
                                for i, k in enumerate(sorted(weights))}}, f)  # fmt: skip
    assert main([partial, *tail]) == 1
    assert "lacks model-00002-of-00002.safetensors" in capsys.readouterr().err
    wider = write_model_dir(str(tmp_path / "wider"), dict(raw, intermediate_size=raw["intermediate_size"] + 16), weights)
    assert main([wider, *tail]) == 1
    err = capsys.readouterr().err
    assert "atomserve:" in err and "mlp.gate_proj.weight" in err and "Traceback" not in err
    other = write_model_dir(str(tmp_path / "other"), dict(raw, architectures=["SomethingElseForCausalLM"]), weights)
    assert main([other, *tail]) == 1
    assert "SomethingElseForCausalLM" in capsys.readouterr().err


def test_engine_thread_under_concurrent_clients(setup):
    """Two seconds of serving on the engine's own thread: clients on eight threads submit prompts
    of all lengths (some share a prefix), stream, and abort now and then, with a pool small
    enough to preempt.  Every request ends as asked or aborted, with as many tokens as it asked
    for; nothing is left running and every page is back."""
    import random
    import threading
    import time

    from atomserve_amd.config import EngineConfig
    from atomserve_amd.engine.engine import create_engine
    from atomserve_amd.engine.sequence import SamplingParams
    from atomserve_amd.weights import load_model

    name, raw, weights, path, _ = setup
    model, _, _ = load_model(path, torch.bfloat16, "cuda:0")
    limit = min(raw["max_position_embeddings"], 200)
    engine = create_engine(model, EngineConfig(block_size=16, num_blocks=40, max_num_seqs=6, max_num_batched_tokens=48,
                                               max_model_len=limit), seed=0)  # fmt: skip
    engine.start()
    stop = time.time() + 2.0
    counts = {"length": 0, "abort": 0}
    problems = []
    lock = threading.Lock()

    def client(i):
        rng = random.Random(i)
        shared = rc.random_ids(raw["vocab_size"], 33, seed=1)
        while time.time() < stop:
            prompt = (shared if rng.random() < 0.4 else []) + rc.random_ids(raw["vocab_size"], rng.randint(1, 90), seed=rng.randrange(1 << 30))
            params = SamplingParams(temperature=rng.choice([0.0, 0.8]), max_tokens=rng.randint(1, 40), ignore_eos=True)
            try:
                handle = engine.submit(prompt, params)
                cut = rng.randint(1, 10) if rng.random() < 0.25 else None
                got = 0
                for _ in handle:
                    got += 1
                    if got == cut:
                        handle.abort()
                with lock:
                    counts[handle.finish_reason] += 1
                    if handle.finish_reason == "length" and got != params.max_tokens:
                        problems.append(f"{got} tokens for max_tokens {params.max_tokens}")
            except Exception as e:  # noqa: BLE001  (reported below, on the main thread)
                with lock:
                    problems.append(repr(e))
                return

    threads = [threading.Thread(target=client, args=(i,)) for i in range(8)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=60)
    assert not any(t.is_alive() for t in threads), "a client never got its last token"
    time.sleep(0.2)
    stats = engine.stats()
    engine.shutdown()
    assert not problems, problems[:3]
    assert counts["length"] > 20 and counts["abort"] > 0
    assert stats["running"] == stats["waiting"] == stats["kv_blocks_used"] == 0


def test_warm_up_captures_the_decode_steps_ahead(setup):
    """After `warm_up` the decode steps of every batch size up to max_num_seqs replay from graphs
    that are already there, and generation gives the plain model's tokens."""
    from atomserve_amd.config import EngineConfig
    from atomserve_amd.engine.engine import create_engine
    from atomserve_amd.engine.sequence import SamplingParams
    from atomserve_amd.weights import load_model

    name, raw, weights, path, _ = setup
    model, _, _ = load_model(path, torch.float32, "cuda:0")
    engine = create_engine(model, EngineConfig(block_size=16, num_blocks=64, max_model_len=128, max_num_seqs=6))
    assert engine.warm_up() == 4  # buckets of 1, 2, 4 and 8 rows
    graphs = engine.runner.decode_graphs.graphs
    assert sorted(graphs) == [(n, 1024) for n in (1, 2, 4, 8)] and engine.warm_up() == 0
    prompts = [rc.random_ids(raw["vocab_size"], n, seed=700 + n) for n in (3, 11, 20, 7, 5)]
    got = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=6, ignore_eos=True))
    assert got == [plain.greedy(raw, weights, p, 6) for p in prompts]
    assert len(graphs) == 4 and engine.stats()["kv_blocks_used"] == 0


def test_a_callers_own_graph_after_the_engines(setup):
    """The engine captures its decode steps under inference mode; a capture that the same process makes
    afterwards outside inference mode (torch fills the random generator's capture state in place, in
    tensors made at the process's first capture) goes through and replays."""
    from atomserve_amd.config import EngineConfig
    from atomserve_amd.engine.engine import create_engine
    from atomserve_amd.weights import load_model

    name, raw, weights, path, _ = setup
    model, _, _ = load_model(path, torch.float32, "cuda:0")
    engine = create_engine(model, EngineConfig(block_size=16, num_blocks=16, max_model_len=64, max_num_seqs=2))
    assert engine.warm_up() == 2
    assert not torch.is_inference_mode_enabled()
    x = torch.zeros(8, device="cuda:0")
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        x += 1
    graph.replay()
    graph.replay()
    torch.cuda.synchronize()
    assert x.tolist() == [2.0] * 8


def test_a_replay_step_that_cannot_run_changes_nothing(setup):
    """A token outside the vocabulary, a wanted place outside its row, a request named twice, a step
    without room: each raises before a page is taken, the requests that were alive keep what they held,
    nobody new is alive, and the trace goes on to the plain model's logits."""
    name, raw, weights, path, cache = setup
    vocab = raw["vocab_size"]
    ids = rc.random_ids(vocab, 40, seed=12)
    replay = make_replay(path, "float32", 128, PAGE[name])
    first = replay.step([{"id": "a", "tokens": ids[:20], "want": [19]}], [])
    held = replay.manager.num_free
    bad_steps = [
        [{"id": "a", "tokens": ids[20:22], "want": [0]}, {"id": "b", "tokens": [1, vocab], "want": [1]}],
        [{"id": "a", "tokens": ids[20:22], "want": [2]}],
        [{"id": "b", "tokens": [1, 2], "want": [-1]}],
        [{"id": "b", "tokens": [1], "want": []}, {"id": "b", "tokens": [2], "want": []}],
        [{"id": "b", "tokens": [1] * 500, "want": []}],
    ]
    for entries in bad_steps:
        with pytest.raises((ValueError, RuntimeError)):
            replay.step(entries, [])
        assert replay.manager.num_free == held and sorted(replay.live) == ["a"] and replay.live["a"][1] == 20
    rest = replay.step([{"id": "a", "tokens": ids[20:], "want": [19]}], ["a"])
    ref = rc.plain_rows(raw, weights, ids, {}, "a", False)
    for got, place in ((first[0], 19), (rest[0], 39)):
        assert float((got - ref[place]).abs().max()) <= rc.TOL_FLOAT32 * max(1.0, float(ref.abs().max()))
    assert replay.manager.num_free == replay.manager.num_blocks and not replay.live


def test_portions_behind_a_long_prefix_cut_their_attention(tmp_path, monkeypatch):
    """Portions of a prompt behind some two thousand cached tokens are few work items of many rounds of keys: the
    prefill attention cuts them along their keys and merges the pieces.  Through the step function, beside another
    request's portion and decoded tokens: every row is the plain model's, within what rounding alone does."""
    from atomserve_amd.kernels import ops

    raw = dict(TINY["B"], max_position_embeddings=4096)
    weights = plain_random_weights(raw, seed=53, std=0.2, gain_std=0.2)
    path = write_model_dir(str(tmp_path / "long"), raw, weights, torch.bfloat16)
    vocab = raw["vocab_size"]
    requests = {"a": rc.random_ids(vocab, 2400, seed=8), "b": rc.random_ids(vocab, 300, seed=9)}
    a, b = requests["a"], requests["b"]
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:1900], "want": [0, 1899]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": a[1900:2030], "want": list(range(0, 130, 9))}], "end": []},
        {"step": 2, "entries": [{"id": "a", "tokens": a[2030:2094], "want": [0, 63]}, {"id": "b", "tokens": b[:200], "want": [199]}], "end": []},
        {"step": 3, "entries": [{"id": "b", "tokens": [b[200]], "want": [0]}, {"id": "a", "tokens": a[2094:2294], "want": list(range(0, 200, 7))}], "end": []},
        {"step": 4, "entries": [{"id": "a", "tokens": a[2294:2303], "want": [8]}, {"id": "b", "tokens": b[201:300], "want": [98]}], "end": ["b"]},
        {"step": 5, "entries": [{"id": "a", "tokens": a[2303:], "want": [0, 96]}], "end": ["a"]},
    ]
    decided = []
    real = ops._prefill_plan
    monkeypatch.setattr(ops, "_prefill_plan", lambda *args, **kw: decided.append(real(*args, **kw)) or decided[-1])
    replay = make_replay(path, "bfloat16", rc.live_token_bound(steps))
    result = compare(replay, steps, requests, raw, weights, {}, "bfloat16", plain_kwargs={"batched": True})
    assert result.rows == 2 + 15 + 3 + 30 + 2 + 2
    # every step's attention had its cut decided, layer by layer: the lone first portion whole, all behind it in pieces
    layers = raw["num_hidden_layers"]
    assert len(decided) == len(steps) * layers
    assert all(pieces == 1 for _, pieces, _ in decided[:layers]) and all(pieces > 1 for _, pieces, _ in decided[layers:])
    assert replay.manager.num_free == replay.manager.num_blocks

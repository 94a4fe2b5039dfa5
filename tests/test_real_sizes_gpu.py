"""Equality with the plain model at the real layer sizes: all 36 layers of Qwen3-8B's sizes with
its whole vocabulary, and the mixed continuous batch at Qwen3-0.6B's sizes, random weights made
on the GPU.  The plain model runs on the GPU too, in float64 and with its attention in matrix
form (tests/test_plain.py holds that form equal to the loops)."""

import random

import pytest
import torch

import bench
from tests import plain_qwen3 as plain
from tests import replay_cases as rc

pytestmark = pytest.mark.gpu

QWEN3_8B = {
    "architectures": ["Qwen3ForCausalLM"], "vocab_size": 151936, "hidden_size": 4096, "intermediate_size": 12288,
    "num_hidden_layers": 36, "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 128,
    "rms_norm_eps": 1e-6, "rope_theta": 1000000.0, "tie_word_embeddings": False, "max_position_embeddings": 40960,
    "hidden_act": "silu",
}  # fmt: skip
QWEN3_06B = {
    "architectures": ["Qwen3ForCausalLM"], "vocab_size": 151936, "hidden_size": 1024, "intermediate_size": 3072,
    "num_hidden_layers": 28, "num_attention_heads": 16, "num_key_value_heads": 8, "head_dim": 128,
    "rms_norm_eps": 1e-6, "rope_theta": 1000000.0, "tie_word_embeddings": True, "max_position_embeddings": 40960,
    "hidden_act": "silu",
}  # fmt: skip
PLAIN = {"dtype": torch.float64, "batched": True}


def device_weights(raw, seed):
    """(architecture, configuration, bfloat16 checkpoint on the GPU, the same numbers in float32)."""
    from atomserve_amd.config.registry import architecture_for
    from atomserve_amd.weights.random_init import random_checkpoint

    arch = architecture_for(raw)
    config = arch.parse_config(raw)
    stored = random_checkpoint(arch, config, seed, dtype=torch.bfloat16, device="cuda:0")
    return arch, config, stored, {k: v.float() for k, v in stored.items()}


def build(arch, config, tensors, dtype):
    from atomserve_amd.models.decoder import DecoderModel
    from atomserve_amd.weights.loader import DictSource, bind_checkpoint

    model = DecoderModel(arch.build_plan(config), dtype, "cuda:0")
    bind_checkpoint(model, arch, config, DictSource(tensors))
    return model


def test_every_layer_of_qwen3_8b_sizes_in_a_mixed_trace():
    """Six requests, four alive at a time, in a pool that holds less than all of them (pages are
    used again): one is cut into portions of several hundred tokens and then decodes from 1,003 to
    1,060 tokens (the split of a long context into partitions, and the second context bucket of
    the replayed decode steps), the others hold 100 to 300 tokens and come and go beside it.  Every
    wanted row against the plain model of the same tensors, in 32-bit and in bfloat16."""
    from atomserve_amd.engine.replay import Replay

    raw = QWEN3_8B
    arch, config, stored, exact = device_weights(raw, seed=5)
    lengths = {"long": 1060, "b": 300, "c": 150, "d": 100, "e": 220, "f": 130}
    requests = {rid: rc.random_ids(raw["vocab_size"], n, seed=50 + i) for i, (rid, n) in enumerate(lengths.items())}
    prompts = {"long": 1003, "b": 280, "c": 120, "d": 60, "e": 200, "f": 100}
    steps = rc.mixed(requests, seed=3, max_live=4, sizes=(300, 257, 64, 190, 33, 2), prompt_lengths=prompts)
    bound = rc.live_token_bound(steps)
    assert bound < sum(-(-n // 64) * 64 for n in lengths.values())
    assert sum(len(s["entries"]) > 1 and any(len(e["tokens"]) > 1 for e in s["entries"])
               and any(len(e["tokens"]) == 1 for e in s["entries"]) for s in steps) > 5  # portions beside decoded tokens
    exact_logits, rounded_logits = {}, {}
    for dtype, tensors in (("float32", exact), ("bfloat16", stored)):
        model = build(arch, config, tensors, getattr(torch, dtype))
        replay = Replay(None, dtype, bound, max_live=4, model=model)
        got = wanted_rows(replay, steps)
        assert replay.manager.num_free == replay.manager.num_blocks
        if dtype == "bfloat16":
            assert len(replay.runner.decode_graphs.graphs) >= 2  # the long request passed a context bucket
        del replay, model
        torch.cuda.empty_cache()
        rows = scale = 0
        err = rc.Spread()  # engine against the exact plain model
        near = rc.Spread()  # engine against the plain model with bfloat16 activations
        noise = rc.Spread()  # what bfloat16 activations alone do to the plain model
        for rid, place, row in got:
            if rid not in exact_logits:
                exact_logits[rid] = plain.logits(raw, exact, requests[rid], **PLAIN).float().cpu()
            want = exact_logits[rid][place]
            err.add(row - want)
            scale = max(scale, float(want.abs().max()))
            rows += 1
            if dtype == "bfloat16":
                if rid not in rounded_logits:
                    rounded_logits[rid] = plain.logits(raw, exact, requests[rid], storage=torch.bfloat16, **PLAIN).float().cpu()
                near.add(row - rounded_logits[rid][place])
                noise.add(rounded_logits[rid][place] - want)
        print(f"{dtype}: {rows} rows, |logits| {scale:.3f}; engine - plain: max {err.worst:.3e} rms {err.rms:.3e}", flush=True)
        assert rows > 150
        if dtype == "float32":
            assert err.worst <= 5e-5 * max(scale, 1.0)
        else:
            print(f"   plain with bfloat16 activations - plain: max {noise.worst:.3e} rms {noise.rms:.3e}; "
                  f"engine - plain with bfloat16 activations: max {near.worst:.3e} rms {near.rms:.3e}", flush=True)
            # The engine is no further from the exact logits than rounding to bfloat16 at the same
            # places takes the plain model itself (root mean square over every logit: a stable
            # figure; the largest of 170 million differences: twice its like).
            assert err.rms <= 1.25 * noise.rms and err.worst <= 2.0 * noise.worst
            assert near.rms <= 1.5 * noise.rms


def wanted_rows(replay, steps):
    """[(request, position in the request, logits row)] of every wanted place of a trace."""
    at, out = {}, []
    for s in steps:
        logits = replay.step(s["entries"], s["end"])
        k = 0
        for e in s["entries"]:
            for w in e["want"]:
                out.append((e["id"], at.get(e["id"], 0) + w, logits[k]))
                k += 1
            at[e["id"]] = at.get(e["id"], 0) + len(e["tokens"])
    return out


def test_the_mixed_batch_of_qwen3_06b_sizes_in_32_bit():
    """The continuous batch of the benchmark at its stated size: 32 requests with prompts of 64 to 2,048
    tokens, half of them sharing their first 32, a budget of 512 tokens a step, 128 tokens decoded each,
    greedy, through scheduler, prefix cache and step function in 32-bit (the analogue of reference
    tests/test_engine.py:106-138 on random weights).  Every generated token is the plain model's best at
    its place (the plain model sees prompt and reply whole, once per request, in float64 on the GPU)."""
    from atomserve_amd.config import EngineConfig
    from atomserve_amd.engine.engine import create_engine
    from atomserve_amd.engine.sequence import SamplingParams

    raw = QWEN3_06B
    arch, config, stored, exact = device_weights(raw, seed=6)
    model = build(arch, config, exact, torch.float32)
    rng = random.Random(0)
    requests, longest, decoded, budget, block = 32, 2048, 128, 512, 16
    prefix = [rng.randrange(raw["vocab_size"]) for _ in range(32)]
    prompts = []
    for i in range(requests):
        body = [rng.randrange(raw["vocab_size"]) for _ in range(rng.randint(64, longest))]
        prompts.append(prefix + body[32:] if i % 2 == 0 else body)
    max_len = longest + decoded + block
    engine = create_engine(model, EngineConfig(block_size=block, num_blocks=requests * max_len // block, max_num_seqs=requests,
                                               max_num_batched_tokens=budget, max_model_len=max_len))  # fmt: skip
    outs = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=decoded, ignore_eos=True))
    stats = engine.stats()
    assert stats["cached_prompt_tokens"] >= 15 * 32 and stats["kv_blocks_used"] == 0
    assert stats["steps"] >= sum(map(len, prompts)) // budget + decoded - 1  # the prompts came in portions beside decoded tokens
    del engine, model
    torch.cuda.empty_cache()
    exact64 = {k: v.double() for k, v in exact.items()}
    for p, out in zip(prompts, outs):
        assert len(out) == decoded
        hidden = plain.hidden_states(raw, exact64, p + out, **PLAIN)[len(p) - 1 : -1]  # the places that chose the reply
        ref = plain.rms_norm(hidden, exact64["model.norm.weight"], raw["rms_norm_eps"]) @ exact64["model.embed_tokens.weight"].T
        best = ref.max(dim=-1).values
        chosen = ref.gather(1, torch.tensor(out, device=ref.device)[:, None])[:, 0]
        # the token is the best one, or ties with it within 32-bit rounding of the logits
        assert float((best - chosen).max()) <= 2e-5 * float(ref.abs().max())


def trace_of_every_route(vocab):
    """Sixty-four short requests and a longer one: their prompts in one step (1,200 rows of the matrix
    products), a portion of 5 tokens beside 64 decoded tokens, a portion of 65 tokens alone (a product of
    65 rows), then decode steps of 64, 32, 16, 12, 8, 3 and 1 rows, two of each, as requests end: every
    way a step's row count chooses the kernels of its matrix products and its attention."""
    rng = random.Random(vocab)
    requests = {f"r{i}": rc.random_ids(vocab, rng.randint(2, 36) + 15, seed=7000 + i) for i in range(64)}
    requests["a"] = rc.random_ids(vocab, 140, seed=6999)
    at = {rid: len(ids) - 15 for rid, ids in requests.items()}
    at["a"] = 70
    steps = [{"step": 0, "end": [], "entries": [{"id": rid, "tokens": ids[: at[rid]], "want": [at[rid] - 1]}
                                                 for rid, ids in requests.items()]}]  # fmt: skip
    alive = [f"r{i}" for i in range(64)]

    def decode(rows, extra=(), end=()):
        entries = list(extra)
        for rid in alive[:rows]:
            entries.append({"id": rid, "tokens": [requests[rid][at[rid]]], "want": [0]})
            at[rid] += 1
        steps.append({"step": len(steps), "entries": entries, "end": list(end)})

    decode(64, extra=[{"id": "a", "tokens": requests["a"][70:75], "want": [0, 4]}])
    steps.append({"step": len(steps), "entries": [{"id": "a", "tokens": requests["a"][75:140], "want": [0, 33, 64]}], "end": ["a"]})
    for rows in (64, 32, 16, 12, 8, 3, 1):
        decode(rows)
        decode(rows)
    steps[-1]["end"] = alive
    return requests, steps


@pytest.mark.parametrize("dtype,products", [("float32", "first"), ("bfloat16", "first"), ("bfloat16", "timed")])
@pytest.mark.parametrize("size", ["0.6b", "1.7b", "4b", "8b", "14b", "32b"])
def test_layer_sizes_of_every_model_the_benchmark_names(size, dtype, products):
    """Two layers of each dense Qwen3 model's sizes that `bench.py` names (widths of 1,024 to 5,120, 16 to 64
    heads in groups of 2 to 8, feed-forwards of 3,072 to 25,600, tied and untied heads over a small vocabulary):
    the sizes choose the kernels (steps a wave of the few-rows products, how K is cut for the split tile product,
    the group of heads that one tile of the decode attention holds), and so do the rows of a step.  Every wanted
    row of a trace that takes each route against the plain model in float64 on the GPU; in bfloat16 with the
    library's first candidates and with the candidates (this package's tile products among them) that timing
    picks, as serving does."""
    from atomserve_amd.config import Qwen3Config
    from atomserve_amd.engine.replay import Replay

    assert set(bench.SIZES) == {"0.6b", "1.7b", "4b", "8b", "14b", "32b"}  # a size added there is added here
    raw = Qwen3Config(**{**bench.SIZES[size], "num_layers": 2, "vocab_size": 5008}).to_dict()
    arch, config, stored, exact = device_weights(raw, seed=17)
    exact64 = {k: v.double() for k, v in exact.items()}
    requests, steps = trace_of_every_route(raw["vocab_size"])
    model = build(arch, config, exact if dtype == "float32" else stored, getattr(torch, dtype))
    replay = Replay(None, dtype, rc.live_token_bound(steps), max_live=65, model=model, fixed_products=products == "first")
    got = wanted_rows(replay, steps)
    chosen = model.env.products.chosen()  # this model's own: no other engine of the process chose for it
    if dtype == "bfloat16":
        assert {rows for rows, _, _, _ in chosen} >= {32, 64} and not model.env.products.trials_pending()
    if products == "first":
        assert set(chosen.values()) <= {0, -1}
    assert replay.manager.num_free == replay.manager.num_blocks and len(got) == 65 + 66 + 3 + 2 * (64 + 32 + 16 + 12 + 8 + 3 + 1)
    assert sorted(n for n, _ in replay.runner.decode_graphs.graphs) == [1, 4, 8, 16, 32, 64]
    err, noise, scale = rc.Spread(), rc.Spread(), 0.0
    logits = {}
    for rid, place, row in got:
        if rid not in logits:
            both = [plain.logits(raw, exact64, requests[rid], **PLAIN).float().cpu()]
            if dtype == "bfloat16":
                both.append(plain.logits(raw, exact64, requests[rid], storage=torch.bfloat16, **PLAIN).float().cpu())
            logits[rid] = both
        want = logits[rid][0][place]
        err.add(row - want)
        scale = max(scale, float(want.abs().max()))
        if dtype == "bfloat16":
            noise.add(logits[rid][1][place] - want)
    print(f"{size} {dtype} {products}: |logits| {scale:.3f}; engine - plain: max {err.worst:.3e} rms {err.rms:.3e}; "
          f"plain with bfloat16 activations - plain: max {noise.worst:.3e} rms {noise.rms:.3e}", flush=True)  # fmt: skip
    if dtype == "float32":
        assert err.worst <= 5e-5 * max(scale, 1.0)
    else:
        assert err.rms <= 1.25 * noise.rms and err.worst <= 2.0 * noise.worst

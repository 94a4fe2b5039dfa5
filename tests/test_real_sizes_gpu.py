"""Equality with the plain model at the real layer sizes: all 36 layers of Qwen3-8B's sizes with
its whole vocabulary, and the mixed continuous batch at Qwen3-0.6B's sizes, random weights made
on the GPU.  The plain model runs on the GPU too, in float64 and with its attention in matrix
form (tests/test_plain.py holds that form equal to the loops)."""

import random

import pytest
import torch

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
        err = Spread()  # engine against the exact plain model
        near = Spread()  # engine against the plain model with bfloat16 activations
        noise = Spread()  # what bfloat16 activations alone do to the plain model
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


class Spread:
    def __init__(self):
        self.worst, self.sum_sq, self.count = 0.0, 0.0, 0

    def add(self, diff):
        self.worst = max(self.worst, float(diff.abs().max()))
        self.sum_sq += float(diff.double().pow(2).sum())
        self.count += diff.numel()

    @property
    def rms(self):
        return (self.sum_sq / max(1, self.count)) ** 0.5


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
    """The continuous batch of the benchmark, smaller: 12 requests with prompts of 64 to 1,024 tokens,
    half of them sharing their first 32, a budget of 512 tokens a step, 24 tokens decoded each, greedy,
    through scheduler, prefix cache and step function in 32-bit.  Every generated token is the plain
    model's best at its place (the plain model sees prompt and reply whole, once per request)."""
    from atomserve_amd.config import EngineConfig
    from atomserve_amd.engine.engine import create_engine
    from atomserve_amd.engine.sequence import SamplingParams

    raw = QWEN3_06B
    arch, config, stored, exact = device_weights(raw, seed=6)
    model = build(arch, config, exact, torch.float32)
    rng = random.Random(0)
    prefix = [rng.randrange(raw["vocab_size"]) for _ in range(32)]
    prompts = []
    for i in range(12):
        body = [rng.randrange(raw["vocab_size"]) for _ in range(rng.randint(64, 1024))]
        prompts.append(prefix + body[32:] if i % 2 == 0 else body)
    decoded = 24
    engine = create_engine(model, EngineConfig(block_size=16, num_blocks=6 * 1100 // 16, max_num_seqs=8,
                                               max_num_batched_tokens=512, max_model_len=1100))  # fmt: skip
    outs = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=decoded, ignore_eos=True))
    stats = engine.stats()
    assert stats["cached_prompt_tokens"] >= 5 * 32 and stats["kv_blocks_used"] == 0
    for p, out in zip(prompts, outs):
        assert len(out) == decoded
        ref = plain.logits(raw, exact, p + out, **PLAIN)[len(p) - 1 : -1]
        best = ref.max(dim=-1).values
        chosen = ref.gather(1, torch.tensor(out, device=ref.device)[:, None])[:, 0]
        # the token is the best one, or ties with it within 32-bit rounding of the logits
        assert float((best - chosen).max()) <= 2e-5 * float(ref.abs().max())

"""Decode and prefill throughput of random-weight Qwen3-8B layer sizes on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--sizes 8b|0.6b|32b] [--batch B] [--context S]
    python bench.py --workload mixed --sizes 0.6b      (a continuous batch through the scheduler)

A step is one decode step of the engine (scheduler, one pass over the GPU, sampling).
Prints ONE JSON line: decoded tokens per second at batch 8 with 2,048-token contexts,
plus prefill of 2,048 tokens, the decode roofline and the batch 1 and 64 points.
Method as in the reference's bench/engine.py: synthetic token ids, prefix caching off,
ignore_eos, warm-up first, prompt steps outside the decode timer, tokens counted.
"""

import argparse
import json
import os
import random
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12  # bytes/s, MI355X HBM3E
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}  # dense MFMA

# Layer sizes by name; "8b" is the configuration the headline number is quoted on.
SIZES = {
    "8b": dict(vocab_size=151936, hidden_size=4096, intermediate_size=12288, num_layers=36, num_heads=32,
               num_kv_heads=8, head_dim=128, rms_norm_eps=1e-6, rope_theta=1e6, tie_word_embeddings=False,
               max_position_embeddings=40960),
    "0.6b": dict(vocab_size=151936, hidden_size=1024, intermediate_size=3072, num_layers=28, num_heads=16,
                 num_kv_heads=8, head_dim=128, rms_norm_eps=1e-6, rope_theta=1e6, tie_word_embeddings=True,
                 max_position_embeddings=40960),
    "32b": dict(vocab_size=151936, hidden_size=5120, intermediate_size=25600, num_layers=64, num_heads=64,
                num_kv_heads=8, head_dim=128, rms_norm_eps=1e-6, rope_theta=1e6, tie_word_embeddings=False,
                max_position_embeddings=40960),
    "1.7b": dict(vocab_size=151936, hidden_size=2048, intermediate_size=6144, num_layers=28, num_heads=16,
                 num_kv_heads=8, head_dim=128, rms_norm_eps=1e-6, rope_theta=1e6, tie_word_embeddings=True,
                 max_position_embeddings=40960),
    "4b": dict(vocab_size=151936, hidden_size=2560, intermediate_size=9728, num_layers=36, num_heads=32,
               num_kv_heads=8, head_dim=128, rms_norm_eps=1e-6, rope_theta=1e6, tie_word_embeddings=True,
               max_position_embeddings=40960),
    "14b": dict(vocab_size=151936, hidden_size=5120, intermediate_size=17408, num_layers=40, num_heads=40,
                num_kv_heads=8, head_dim=128, rms_norm_eps=1e-6, rope_theta=1e6, tie_word_embeddings=False,
                max_position_embeddings=40960),
}  # fmt: skip


def parse_args():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=256, help="decode steps timed: every sequence generates this many tokens")
    p.add_argument("--warmup", type=int, default=8)
    p.add_argument("--batch", type=int, default=8)
    p.add_argument("--context", type=int, default=2048)
    p.add_argument("--shortest-context", type=int, default=0, help="contexts spread evenly from this many tokens to "
                   "--context over the batch instead of all equal (0: equal)")
    p.add_argument("--sizes", choices=sorted(SIZES), default="8b", help="layer sizes of a dense Qwen3 model")
    p.add_argument("--layers", type=int, default=None, help="fewer layers than the model has (both counts are reported)")
    p.add_argument("--max-len", type=int, default=4096, help="longest sequence the cache pool is sized for")
    p.add_argument("--dtype", choices=["bf16", "fp32"], default="bf16")
    p.add_argument("--points", default="1,64", help="other decode batch sizes to measure (fewer steps each)")
    p.add_argument("--block-size", type=int, default=16, help="tokens per cache page")
    p.add_argument("--no-prefill", action="store_true")
    p.add_argument("--prefill-tokens", type=int, default=2048, help="length of the prompt whose prefill is timed "
                   "(longer than the step budget: in portions of it)")  # fmt: skip
    p.add_argument("--budget", type=int, default=None, help="token budget of a step (default: 2,048, or --context if that "
                   "is more): prompts longer than this are prefilled in portions of it")  # fmt: skip
    p.add_argument("--no-calibration", action="store_true", help="skip the library copy and matmul probes")
    p.add_argument("--greedy", action="store_true", help="greedy instead of the default sampling settings")
    p.add_argument("--workload", choices=["decode", "mixed"], default="decode",
                   help="decode: the timed decode steps above; mixed: 32 requests with prompts of 64 to 2,048 tokens "
                        "(half of them share their first 32), chunks of 512, 128 tokens decoded each, through the "
                        "scheduler from submission to the last token")  # fmt: skip
    p.add_argument("--chunk-budget", type=int, default=512, help="token budget of a step in the mixed workload")
    p.add_argument("--profile", action="store_true",
                   help="also split the host's time of a decode step into schedule / pack / launch / sample / wait / "
                        "update (steps run one at a time meanwhile, none sent ahead), as the reference's "
                        "bench/engine.py --profile does")  # fmt: skip
    return p.parse_args()


def prompt(b: int, n: int, vocab: int) -> list:
    """Distinct synthetic prompts (reference bench/engine.py:90-92)."""
    return [(1000 + 37 * b + i) % (vocab - 1000) for i in range(n)]


def mixed_workload(args, model, config, full_layers: int) -> dict:
    """A continuous batch as a server sees it: everything is submitted at once, prompts are cut
    into portions under the token budget beside the running requests' decode steps, prefixes are
    reused.  One untimed run first (graphs are captured, libraries pick their kernels), then the
    median of three runs with other prompts of the same lengths' distribution."""
    import random

    import torch

    from atomserve_amd.config import EngineConfig
    from atomserve_amd.engine.engine import create_engine
    from atomserve_amd.engine.sequence import SamplingParams

    requests, longest, decoded, budget, block = 32, 2048, 128, args.chunk_budget, 16
    max_len = longest + decoded + block
    engine = create_engine(model, EngineConfig(block_size=block, num_blocks=requests * max_len // block,
                                               max_num_seqs=requests, max_num_batched_tokens=budget,
                                               max_model_len=max_len, enable_prefix_caching=True), seed=0)  # fmt: skip
    engine.warm_up()  # as the command line does before it serves
    params = SamplingParams(temperature=0.0, max_tokens=decoded, ignore_eos=True) if args.greedy else \
        SamplingParams(max_tokens=decoded, ignore_eos=True)  # fmt: skip
    rng = random.Random(0)

    def run():
        prefix = [rng.randrange(1000, config.vocab_size - 1000) for _ in range(32)]
        prompts = []
        for i in range(requests):
            body = [rng.randrange(1000, config.vocab_size - 1000) for _ in range(rng.randint(64, longest))]
            prompts.append(prefix + body[32:] if i % 2 == 0 else body)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for p in prompts:
            engine.submit(p, params)
        steps = 0
        while engine.step():
            steps += 1
        torch.cuda.synchronize()
        return time.perf_counter() - t0, sum(map(len, prompts)), steps

    run()
    dt, prompt_tokens, steps = sorted(run() for _ in range(3))[1]
    c = config
    return {
        "metric": f"generated tok/s of a mixed continuous batch (Qwen3-{args.sizes.upper()} sizes, random weights)",
        "value": round(requests * decoded / dt, 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": 1,
        "ms_per_step": round(dt / steps * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": args.dtype,
        "data": "synthetic token ids, random-init weights",
        "config": {
            "model": f"Qwen3-{args.sizes.upper()} sizes", "layers": c.num_layers, "layers_full": full_layers,
            "hidden": c.hidden_size, "heads": c.num_heads, "kv_heads": c.num_kv_heads, "head_dim": c.head_dim,
            "intermediate": c.intermediate_size, "vocab": c.vocab_size, "global_batch": requests,
            "seq_len": longest, "decoded_each": decoded, "chunk_budget": budget, "block_size": block,
            "shared_prefix": 32, "parallelism": "single GPU",
            "sampling": "greedy" if args.greedy else "temperature 0.6 top-k 20 top-p 0.95",
        },
        "run_ms": round(dt * 1e3, 1),
        "prompt_tokens": prompt_tokens,
        "all_tokens_per_s": round((prompt_tokens + requests * decoded) / dt, 1),
    }


def calibrate(device) -> dict:
    """What this GPU delivers to plain library calls, to read the roofline fractions against: a
    1 GiB device copy (bytes read plus written per second) and an 8192^3 bf16 matrix product."""
    import torch

    def timed(fn, n=5):
        fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / n

    x = torch.empty(1 << 30, dtype=torch.uint8, device=device)
    y = torch.empty_like(x)
    copy = 2 * x.numel() / timed(lambda: y.copy_(x))
    a = torch.randn(8192, 8192, device=device).to(torch.bfloat16)
    b = torch.randn(8192, 8192, device=device).to(torch.bfloat16)
    matmul = 2 * 8192**3 / timed(lambda: torch.mm(a, b.t()))
    return {"copy_GBps": round(copy / 1e9, 1), "matmul_bf16_TFLOPs": round(matmul / 1e12, 1)}


def main() -> int:
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported (this engine runs on a single MI355X)")
        return 2

    import torch

    from atomserve_amd.config import EngineConfig, Qwen3Config
    from atomserve_amd.config.registry import architecture_for
    from atomserve_amd.engine.engine import create_engine
    from atomserve_amd.engine.sequence import SamplingParams
    from atomserve_amd.models.decoder import DecoderModel
    from atomserve_amd.weights.loader import DictSource, bind_checkpoint
    from atomserve_amd.weights.random_init import random_checkpoint

    device = "cuda:0"
    dtype = torch.bfloat16 if args.dtype == "bf16" else torch.float32
    calibration = None if args.no_calibration else calibrate(device)
    full_layers = SIZES[args.sizes]["num_layers"]
    config = Qwen3Config(**{**SIZES[args.sizes], "num_layers": args.layers or full_layers})
    arch = architecture_for(config.to_dict())
    model = DecoderModel(arch.build_plan(config), dtype, device)
    bind_checkpoint(model, arch, config, DictSource(random_checkpoint(arch, config, seed=0, dtype=dtype, device=device)))
    torch.cuda.synchronize()
    if args.workload == "mixed":
        print(json.dumps(mixed_workload(args, model, config, full_layers)))
        return 0

    batches = sorted({args.batch, *[int(b) for b in args.points.split(",") if b]})
    block = args.block_size
    max_len = max(args.max_len, args.context + args.steps + args.warmup + 16 + (64 if args.profile else 0),
                  args.prefill_tokens + 16)
    num_blocks = max(batches) * -(-max_len // block)
    params = SamplingParams(temperature=0.0, max_tokens=100000, ignore_eos=True) if args.greedy else \
        SamplingParams(max_tokens=100000, ignore_eos=True)  # fmt: skip
    engine_config = EngineConfig(block_size=block, num_blocks=num_blocks, max_num_seqs=max(batches),
                                 max_num_batched_tokens=args.budget or max(2048, args.context), max_model_len=max_len,
                                 enable_prefix_caching=False)  # fmt: skip
    engine = create_engine(model, engine_config, seed=0)
    engine.warm_up()  # as the command line does before it serves: decode steps captured, prompt lengths tried

    itemsize = 2 if args.dtype == "bf16" else 4
    c = config
    layer_params = c.hidden_size * (c.num_heads + 2 * c.num_kv_heads) * c.head_dim + c.num_heads * c.head_dim * c.hidden_size \
        + 3 * c.hidden_size * c.intermediate_size  # fmt: skip
    weight_bytes = (layer_params * c.num_layers + c.vocab_size * c.hidden_size) * itemsize
    kv_bytes_per_token = c.num_layers * 2 * c.num_kv_heads * c.head_dim * itemsize

    host_phases = {}

    def roofline(batch: int, mean_ctx: float, ms: float) -> dict:
        """The bytes a decode step has to read (every weight once, the cache of the live requests)
        over its time, against the HBM peak."""
        achieved = (weight_bytes + batch * mean_ctx * kv_bytes_per_token) / (ms * 1e-3)
        return {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK, 4)}  # fmt: skip

    def run_decode(batch: int, steps: int, warmup: int, profile: int = 0):
        """Prefill `batch` prompts of args.context tokens (untimed), then time `steps` decode steps."""
        lo = args.shortest_context or args.context
        lengths = [lo + (args.context - lo) * b // max(1, batch - 1) for b in range(batch)]
        random.Random(0).shuffle(lengths)
        handles = [engine.submit(prompt(b, n, c.vocab_size), params) for b, n in enumerate(lengths)]
        while any(s.num_computed_tokens < s.num_prompt_tokens for s in
                  [*engine.scheduler.running, *engine.scheduler.waiting]) or engine.scheduler.waiting or not engine.scheduler.running:
            engine.step()
        for _ in range(warmup):
            engine.step()
        ctx_start = sum(s.num_tokens for s in engine.scheduler.running) / batch
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            engine.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        assert len(engine.scheduler.running) == batch and engine.last_batch_tokens == batch
        mean_ctx = ctx_start + steps / 2
        if profile:
            phases = engine.profile_phases(True)
            for _ in range(profile):
                engine.step()
            engine.profile_phases(False)
            host_phases.update(phases.mean_us())
        for h in handles:
            engine.abort(h.id)
        engine.step()
        assert engine.stats()["kv_blocks_used"] == 0
        return batch * steps / dt, dt / steps * 1e3, mean_ctx

    result_prefill = None
    if not args.no_prefill:
        one = SamplingParams(temperature=0.0, max_tokens=1, ignore_eos=True)
        T = args.prefill_tokens
        for i in range(2):  # warm-up: libraries pick their kernels, pools are touched
            engine.generate([prompt(99 - i, T, c.vocab_size)], one)
        times = []
        for i in range(3):  # different prompts, nothing reused; the median of three
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            engine.generate([prompt(90 + i, T, c.vocab_size)], one)
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t0)
        dt = sorted(times)[1]
        flops = 2 * T * layer_params * c.num_layers + 2 * c.hidden_size * c.vocab_size \
            + 4 * c.num_heads * c.head_dim * (T * (T + 1) // 2) * c.num_layers  # fmt: skip
        result_prefill = {"value": round(T / dt, 1), "tokens": T, "ms": round(dt * 1e3, 3),
                          "frac": round(flops / dt / PEAK_FLOPS[args.dtype], 4)}  # fmt: skip

    points, point_rooflines = {}, {}
    for b in batches:
        if b != args.batch:
            tps, ms, ctx = run_decode(b, max(16, args.steps // 4), max(2, args.warmup // 2))
            points[f"decode_b{b}"] = round(tps, 1)
            point_rooflines[f"decode_b{b}"] = roofline(b, ctx, ms)
    tps, ms, mean_ctx = run_decode(args.batch, args.steps, args.warmup, profile=64 if args.profile else 0)

    line = {
        "metric": f"decode tok/s at batch {args.batch}, {args.context}-token contexts (Qwen3-{args.sizes.upper()} sizes, random weights)",
        "value": round(tps, 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": args.dtype,
        "data": "synthetic token ids, random-init weights",
        "config": {
            "model": f"Qwen3-{args.sizes.upper()} sizes", "layers": c.num_layers, "layers_full": full_layers, "hidden": c.hidden_size,
            "heads": c.num_heads, "kv_heads": c.num_kv_heads, "head_dim": c.head_dim,
            "intermediate": c.intermediate_size, "vocab": c.vocab_size, "global_batch": args.batch,
            "seq_len": args.context, "shortest_context": args.shortest_context or args.context, "max_context": max_len, "block_size": block,
            "step_budget": engine_config.max_num_batched_tokens, "parallelism": "single GPU",
            "sampling": "greedy" if args.greedy else "temperature 0.6 top-k 20 top-p 0.95",
        },
        "roofline": roofline(args.batch, mean_ctx, ms),
        "points": points,
        "roofline_points": point_rooflines,
    }
    if host_phases:
        line["host_phases_us"] = host_phases
        print("host time of a decode step without steps sent ahead, microseconds: "
              + ", ".join(f"{k} {v}" for k, v in host_phases.items()), file=sys.stderr)  # fmt: skip
    if result_prefill:
        line["prefill"] = result_prefill
    if calibration:
        line["calibration"] = calibration
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())

"""Command line: `atomserve <model folder>` (reference atomserve/cli.py:34-204).

    load config + weights  ->  size the cache pool  ->  build the engine  ->  warm up
    ->  generate for the given prompts (token ids), or read prompts line by line

Option names and meanings follow the reference where it has them (--dtype, --kv-mem-gb,
--block-size, --max-num-seqs, --max-batched-tokens, --no-prefix-caching, --version).
The engine deals in token ids only, so prompts are given as ids; the HTTP server, the
chat REPL and the tokenizer of the reference are not part of this engine.
"""

import argparse
import json
import os
import sys
import time

from atomserve_amd import __version__

DTYPES = ("bf16", "fp32")


def kv_budget(text: str):
    """--kv-mem-gb: a number of GiB, or 'auto'."""
    if text.strip().lower() == "auto":
        return "auto"
    try:
        value = float(text)
    except ValueError:
        raise argparse.ArgumentTypeError(f"{text!r} is neither a number of GiB nor 'auto'") from None
    if value <= 0:
        raise argparse.ArgumentTypeError("the KV cache needs a positive amount of memory")
    return value


def fit_kv_budget(wanted, free_bytes: int, reserve_bytes: int, note=print) -> float:
    """The GiB the cache pool gets: what was asked for, cut down to what the GPU has free after
    the weights minus a reserve for a step's activations, its logits and the libraries' workspaces
    (the reference shrinks its budget the same way on its device, atomserve/cli.py:122-136).
    'auto' takes all of that room.  Exits with a message when no room worth a pool is left."""
    room = (free_bytes - reserve_bytes) / 2**30
    if room < 0.25:
        raise SystemExit(
            f"atomserve: the weights leave {free_bytes / 2**30:.1f} GiB of GPU memory free, of which "
            f"{reserve_bytes / 2**30:.1f} GiB are kept for activations: no room for a KV cache "
            "(a smaller model, or --dtype bf16, leaves more)"
        )
    if wanted == "auto":
        return room
    if wanted > room:
        note(f"Note: KV cache reduced from {wanted:.1f} to {room:.1f} GiB to fit in GPU memory.")
        return room
    return float(wanted)


def step_reserve_bytes(plan, max_batched_tokens: int, max_num_seqs: int) -> int:
    """Memory a step needs beside weights and cache, generously: the rows of a full step in every
    width a layer makes of them, the logits of the replayed decode steps, and the libraries."""
    widest = 0
    for layer in plan.layers:
        mixer, ffn = layer.mixer, layer.ffn
        heads = getattr(mixer, "num_heads", 0) + 2 * getattr(mixer, "num_kv_heads", 0)
        widest = max(widest, 8 * plan.hidden_size + 8 * heads * getattr(mixer, "head_dim", 0)
                     + 12 * getattr(ffn, "intermediate_size", plan.hidden_size))  # fmt: skip
    logits = 4 * plan.vocab_size * (2 * min(256, max_num_seqs) + 64)
    return (1 << 30) + 2 * max_batched_tokens * widest + logits


def build_parser() -> argparse.ArgumentParser:
    p = argparse.ArgumentParser(
        prog="atomserve",
        description="Run a Qwen3 model folder on one MI355X and generate from token-id prompts.",
        formatter_class=argparse.ArgumentDefaultsHelpFormatter,
    )
    p.add_argument("model", help="local model directory (config.json + *.safetensors); with --random-weights, "
                                 "a directory or file holding only config.json")  # fmt: skip
    p.add_argument("--dtype", choices=DTYPES, default="bf16", help="weights, activations and the KV cache")
    p.add_argument("--kv-mem-gb", type=kv_budget, default=4.0,
                   help="GiB of memory for the KV cache, or 'auto' for all that the weights leave free; "
                        "reduced with a note if the GPU has less left")  # fmt: skip
    p.add_argument("--block-size", type=int, default=16, help="tokens per KV block")
    p.add_argument("--max-num-seqs", type=int, default=32, help="most requests running at once")
    p.add_argument("--max-batched-tokens", type=int, default=512,
                   help="token budget of one forward pass; smaller bounds the stall a long prompt causes "
                        "running streams, larger prefills faster (on an MI355X 2048 gives a mixed batch of "
                        "Qwen3-8B size a fifth more throughput than 512, for steps of 28 ms instead of 12)")  # fmt: skip
    p.add_argument("--no-prefix-caching", action="store_true", help="always recompute shared prompt prefixes")
    p.add_argument("--max-model-len", type=int, default=None, help="longest sequence accepted (default: what model and pool allow)")
    p.add_argument("--random-weights", type=int, default=None, metavar="SEED",
                   help="ignore any weight files and draw random weights from this seed")  # fmt: skip
    p.add_argument("--prompt-ids", action="append", default=[], metavar="IDS",
                   help="a prompt as comma- or space-separated token ids; may be given several times")  # fmt: skip
    p.add_argument("--prompt-file", help="file with one prompt per line, as token ids")
    p.add_argument("--max-tokens", type=int, default=64, help="tokens to generate per prompt")
    p.add_argument("--temperature", type=float, default=0.6, help="0 is greedy")
    p.add_argument("--top-k", type=int, default=20, help="sample among the k most likely tokens; 0 disables")
    p.add_argument("--top-p", type=float, default=0.95, help="then among the smallest set reaching this mass")
    p.add_argument("--presence-penalty", type=float, default=0.0, help="subtracted from logits of generated tokens")
    p.add_argument("--seed", type=int, default=None, help="fixed seed for reproducible sampling")
    p.add_argument("--ignore-eos", action="store_true", help="keep generating past end-of-sequence")
    p.add_argument("--fixed-products", action="store_true",
                   help="always take the library's first candidate for its matrix products instead of timing them at "
                        "start-up: bfloat16 results are then the same from run to run (a little slower at 17 to 64 "
                        "requests and for prompts)")  # fmt: skip
    p.add_argument("--no-stream-copies", action="store_true",
                   help="do not keep the weights a second time in the order the decode kernels read them: saves "
                        "their bytes again (15 GB at Qwen3-8B sizes), decode steps are some 7 per cent slower")  # fmt: skip
    p.add_argument("--version", action="version", version=f"%(prog)s {__version__}")
    return p


def engine_config_for(args, bytes_per_block: int, max_positions: int):
    """Size the pool from the memory budget; cap the sequence length by pool and model
    (reference atomserve/cli.py:99-119)."""
    from atomserve_amd.config import EngineConfig

    if args.kv_mem_gb == "auto":
        raise ValueError("the budget must be fitted to the GPU first (fit_kv_budget)")
    num_blocks = int(args.kv_mem_gb * 2**30 // bytes_per_block)
    if num_blocks < 1:
        raise SystemExit("atomserve: --kv-mem-gb leaves no room for a single KV block")
    limit = min(max_positions, num_blocks * args.block_size)
    if args.max_model_len is not None:
        limit = min(limit, args.max_model_len)
    try:
        return EngineConfig(
            block_size=args.block_size,
            num_blocks=num_blocks,
            max_num_seqs=args.max_num_seqs,
            max_num_batched_tokens=args.max_batched_tokens,
            max_model_len=limit,
            enable_prefix_caching=not args.no_prefix_caching,
        )
    except ValueError as error:  # limits that contradict each other: a message, not a traceback
        raise SystemExit(f"atomserve: {error}") from None


def parse_ids(text: str) -> list:
    return [int(t) for t in text.replace(",", " ").split()]


def eos_ids(model_dir: str) -> frozenset:
    """End-of-sequence ids from generation_config.json, if the folder has one
    (the reference takes them from there through its tokenizer, atomserve/tokenizer.py:35-38)."""
    path = os.path.join(model_dir, "generation_config.json")
    if not os.path.isfile(path):
        return frozenset()
    with open(path) as f:
        eos = json.load(f).get("eos_token_id", [])
    return frozenset(eos if isinstance(eos, list) else [eos])


def main(argv=None) -> int:
    args = build_parser().parse_args(argv)
    start = time.perf_counter()

    import torch

    from atomserve_amd.cache.pools import CachePools
    from atomserve_amd.config.registry import architecture_for
    from atomserve_amd.engine.engine import create_engine
    from atomserve_amd.engine.sequence import SamplingParams
    from atomserve_amd.models.decoder import DecoderModel
    from atomserve_amd.weights.loader import DictSource, bind_checkpoint, load_weights
    from atomserve_amd.weights.random_init import random_checkpoint

    if not torch.cuda.is_available():
        print("atomserve: no GPU is visible; this engine runs on an MI355X only.", file=sys.stderr)
        return 1
    model_dir = args.model if os.path.isdir(args.model) else os.path.dirname(args.model) or "."
    config_path = os.path.join(model_dir, "config.json") if os.path.isdir(args.model) else args.model
    if not os.path.isfile(config_path):
        print(f"atomserve: no config.json at {config_path}", file=sys.stderr)
        return 1
    dtype = torch.bfloat16 if args.dtype == "bf16" else torch.float32
    try:  # what is wrong with the folder is a message, not a traceback
        with open(config_path) as f:
            raw = json.load(f)
        arch = architecture_for(raw)
        config = arch.parse_config(raw)
        print(f"Loading {args.model} ({args.dtype}, {arch.name}) ...", file=sys.stderr, flush=True)
        model = DecoderModel(arch.build_plan(config), dtype, "cuda:0", stream_copies=not args.no_stream_copies)
        if args.random_weights is not None:
            source = DictSource(random_checkpoint(arch, config, args.random_weights, dtype=dtype, device="cuda:0"))
            bind_checkpoint(model, arch, config, source, where="(random)")
        else:
            load_weights(model_dir, model, arch, config)
    except (FileNotFoundError, ValueError) as error:  # a missing file, a config or a checkpoint that does not fit
        print(f"atomserve: {error}", file=sys.stderr)
        return 1
    block_bytes = CachePools.bytes_per_block(model.cache_requests(), args.block_size, dtype) or 1
    torch.cuda.synchronize()
    torch.cuda.empty_cache()  # what loading used for conversions counts as free
    free_bytes, _ = torch.cuda.mem_get_info()
    args.kv_mem_gb = fit_kv_budget(args.kv_mem_gb, free_bytes,
                                   step_reserve_bytes(model.plan, args.max_batched_tokens, args.max_num_seqs),
                                   note=lambda text: print(text, file=sys.stderr, flush=True))  # fmt: skip
    if args.kv_mem_gb * 2**30 // block_bytes > 2**31 // args.block_size:  # slots are 32-bit integers
        args.kv_mem_gb = (2**31 // args.block_size) * block_bytes / 2**30
    engine_config = engine_config_for(args, block_bytes, model.plan.max_positions)
    model.env.products.fix(args.fixed_products)
    engine = create_engine(model, engine_config, eos_ids(model_dir), seed=args.seed)
    engine.generate([[0]], SamplingParams(temperature=0.0, max_tokens=2, ignore_eos=True))  # compile and warm up
    engine.warm_up()  # and capture the decode steps of every batch size now, not at their first use
    print(
        f"Ready in {time.perf_counter() - start:.1f}s. KV cache: "
        f"{engine_config.num_blocks * engine_config.block_size:,} tokens, context up to {engine_config.max_model_len:,}; "
        f"captured decode steps hold {engine.stats().get('graph_bytes', 0) / 2**20:,.0f} MiB.",
        file=sys.stderr, flush=True,
    )  # fmt: skip

    try:
        params = SamplingParams(temperature=args.temperature, top_k=args.top_k, top_p=args.top_p,
                                presence_penalty=args.presence_penalty, max_tokens=args.max_tokens, seed=args.seed,
                                ignore_eos=args.ignore_eos).validated()  # fmt: skip
    except ValueError as error:
        raise SystemExit(f"atomserve: {error}") from None
    prompts = [parse_ids(p) for p in args.prompt_ids]
    if args.prompt_file:
        with open(args.prompt_file) as f:
            prompts += [parse_ids(line) for line in f if line.strip()]

    def run(batch):
        handles = [engine.submit(p, params) for p in batch]
        while engine.step():
            pass
        for h in handles:
            tokens = list(h)
            print(json.dumps({"prompt_tokens": h.num_prompt_tokens, "output_ids": tokens,
                              "finish_reason": h.finish_reason, "cached_tokens": h.num_cached_tokens}), flush=True)  # fmt: skip

    if prompts:
        run(prompts)
    else:
        print("Enter a prompt as token ids per line, Ctrl-D to exit.", file=sys.stderr, flush=True)
        for line in sys.stdin:
            if line.strip():
                try:
                    run([parse_ids(line)])
                except ValueError as error:
                    print(f"atomserve: {error}", file=sys.stderr, flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())

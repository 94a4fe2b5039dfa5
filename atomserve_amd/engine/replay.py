"""Trace replay: feed given token ids through the model step by step and write logits.

It samples nothing and has no forward pass, cache or loader of its own: it loads the
model as the engine does, takes pages from the engine's cache manager and calls the
engine's step function (`ModelRunner.step`), so what it measures is what generation
runs.  The reference's nearest pieces are `ModelRunner.run` for tools and the
`full_logits` fixture (atomserve/runner.py:182-192, tests/conftest.py:79-98); its
mixed-batch test names the cache geometry (4-token pages, pages handed out in turn)
beside the steps (tests/test_runner.py:103-141), and so does a trace here.

Input, one JSON object per line on standard input:

    {"geometry": {"block_size": 8, "pages": 40, "max_live": 4}}                    (optional, first)
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

`geometry` names the cache: tokens per page, pages in the pool, most requests alive at
once; each key is optional and overrides the command line's --block-size, --pages and
--max-live.  Without a page count the pool holds what --max-tokens asks for.
`entries` are one batch: each request's next tokens and the places among them whose
logits are wanted.  `end` lists requests finished after the step; their pages return
to the pool.  For a step with wanted places `<out>/<step>.f32` receives the logits as
little-endian float32 [wanted, vocab], in the order of the entries and of `want`.
After every step `done <step>` is printed and flushed.

bfloat16 results are those of the kernels serving uses.  Steps of more than 16 rows and
portions of prompts multiply through the library's matrix products; here the library's
first candidate is always taken, so two runs of a trace agree bit for bit.  A serving
engine times the candidates and may settle on another; --timed-products does the same.
"""

import argparse
import json
import os
import sys

DTYPES = {"bfloat16": "bfloat16", "bf16": "bfloat16", "float32": "float32", "fp32": "float32"}
ROUNDING = 64  # --max-tokens counts each live request's tokens rounded up to this


def pages_for(max_tokens: int, block_size: int, max_live: int) -> int:
    """Pages that hold `max_tokens` tokens of up to `max_live` requests, each request's count
    rounded up to 64: exactly max_tokens / block_size where pages divide 64 tokens, else one page
    more per request for the page each may leave partly empty beyond its rounded count."""
    pages = -(-max_tokens // block_size)
    if ROUNDING % block_size:
        pages += max_live
    return max(1, pages)


class Replay:
    def __init__(self, model_dir: str, dtype: str, max_tokens: int = 0, device: str = "cuda:0", log=None,
                 block_size: int = 16, num_pages: int = None, max_live: int = 8, fixed_products: bool = True,
                 model=None):  # fmt: skip
        """model: a model built and bound already (weights made in memory); `model_dir` is then unused."""
        import torch

        from atomserve_amd.cache.manager import CacheManager
        from atomserve_amd.engine.runner import ModelRunner
        from atomserve_amd.weights.loader import load_model

        self.log = log or (lambda msg: None)
        if block_size < 1 or max_live < 1:
            raise ValueError("block size and live-request limit must be positive")
        if num_pages is None:
            num_pages = pages_for(max_tokens, block_size, max_live)
        if num_pages < 1:
            raise ValueError("the cache pool needs at least one page")
        torch_dtype = getattr(torch, DTYPES[dtype])
        if model is not None:
            if model.env.dtype != torch_dtype:
                raise ValueError(f"the model computes in {model.env.dtype}, the replay was asked for {torch_dtype}")
            self.model = model
        else:
            self.log(f"loading {model_dir} ({DTYPES[dtype]}) ...")
            self.model, self.arch, self.config = load_model(model_dir, torch_dtype, device)
        self.model.env.products.fix(fixed_products)  # this model's products only: another engine of the process keeps its own
        self.block_size, self.max_live = block_size, max_live
        self.manager = CacheManager(self.model.cache_requests(), block_size, num_pages, max_live)
        self.runner = ModelRunner(self.model, self.manager)
        self.live: dict = {}  # request id -> [RequestCache, tokens computed so far]
        self.log(f"cache: {num_pages} pages of {block_size} tokens, up to {max_live} live requests")

    def step(self, entries: list, end: list):
        """Run one step; returns the logits of its wanted places as a CPU tensor, or None.
        A step that cannot run (a token outside the vocabulary, a wanted place outside its row, no room,
        too many requests) raises before anything is taken and changes nothing.  If the pass itself
        fails on the GPU, the requests that this step started are dropped with their pages, and the
        pages it added to older requests stay theirs (they are given back when those requests end)."""
        from atomserve_amd.engine.batch import Row

        work, seen = [], set()
        vocab = self.runner.vocab_size
        for e in entries:
            rid, tokens, want = e["id"], [int(t) for t in e["tokens"]], [int(w) for w in e.get("want", [])]
            if rid in seen:
                raise ValueError(f"request {rid!r} appears twice in one step")
            seen.add(rid)
            if not tokens:  # an entry that brings nothing runs nothing
                if want:
                    raise ValueError(f"request {rid!r} wants logits of a step in which it has no tokens")
                continue
            outside = [t for t in tokens if not 0 <= t < vocab]
            if outside:
                raise ValueError(f"request {rid!r}: token id {outside[0]} is outside the vocabulary of {vocab}")
            if any(not 0 <= w < len(tokens) for w in want):
                raise ValueError(f"request {rid!r} wants logits at places {want} outside its {len(tokens)} tokens")
            work.append((rid, tokens, want))
        fresh = [rid for rid, _, _ in work if rid not in self.live]
        if len(self.live) + len(fresh) > self.max_live:
            raise RuntimeError(f"more than {self.max_live} requests would be alive; raise --max-live")
        started = {rid: [self.manager.new_request(), 0] for rid in fresh}
        state_of = lambda rid: self.live.get(rid) or started[rid]  # noqa: E731
        if not self.manager.reserve_all([(state_of(rid)[0], state_of(rid)[1], len(tokens)) for rid, tokens, _ in work]):
            raise RuntimeError(
                f"the cache pool ({self.manager.num_blocks} pages of {self.block_size} tokens, "
                f"{self.manager.num_free} free) has no room for this step's "
                f"{sum(len(t) for _, t, _ in work)} tokens; --max-tokens or --pages is too small for the live requests"
            )
        self.live.update(started)
        rows = [Row(tokens, self.live[rid][1], self.live[rid][0].tables, want, self.live[rid][0].state_slot)
                for rid, tokens, want in work]  # fmt: skip
        logits = None
        if rows:
            try:
                out = self.runner.step(rows)
            except BaseException:
                for rid in started:
                    self.manager.release(self.live.pop(rid)[0])
                raise
            if out.shape[0]:
                logits = out.cpu()
            for rid, tokens, _ in work:
                state = self.live[rid]
                state[1] += len(tokens)
                self.manager.release_behind_window(state[0], state[1])
        for rid in end:
            if rid in self.live:
                self.manager.release(self.live.pop(rid)[0])
        return logits


def build_parser() -> argparse.ArgumentParser:
    p = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0],
                                epilog="bfloat16 runs are reproducible from run to run unless --timed-products "
                                       "is given (then the library's matrix-product candidates are timed, as a "
                                       "serving engine does, and the winner may differ between runs).")  # fmt: skip
    p.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    p.add_argument("--dtype", required=True, choices=sorted(DTYPES), help="bfloat16: what serving uses; float32: true 32-bit")
    p.add_argument("--out", required=True, help="folder for <step>.f32 files")
    p.add_argument("--max-tokens", type=int, default=None,
                   help="most tokens that live requests hold at any time, each request's count rounded up to 64")  # fmt: skip
    p.add_argument("--block-size", type=int, default=16, help="tokens per cache page")
    p.add_argument("--pages", type=int, default=None, help="pages in the cache pool (default: what --max-tokens needs)")
    p.add_argument("--max-live", type=int, default=8, help="most requests alive at once")
    p.add_argument("--timed-products", action="store_true",
                   help="let the library's matrix products be chosen by timing, as in serving")  # fmt: skip
    p.add_argument("--device", default="cuda:0", help=argparse.SUPPRESS)
    return p


def main(argv=None, stdin=None) -> int:
    parser = build_parser()
    args = parser.parse_args(argv)
    stdin = stdin or sys.stdin

    def log(msg):
        print(f"trace_run: {msg}", file=sys.stderr, flush=True)

    os.makedirs(args.out, exist_ok=True)
    replay = None
    for line in stdin:
        line = line.strip()
        if not line:
            continue
        record = json.loads(line)
        if replay is None:
            geometry = record.get("geometry", {}) if "step" not in record else {}
            unknown = set(geometry) - {"block_size", "pages", "max_live"}
            if unknown:
                parser.error(f"unknown geometry keys {sorted(unknown)}")
            block_size = int(geometry.get("block_size", args.block_size))
            pages = geometry.get("pages", args.pages)
            if pages is None and args.max_tokens is None:
                parser.error("one of --max-tokens, --pages or a geometry line with pages is needed")
            replay = Replay(args.model, args.dtype, args.max_tokens or 0, device=args.device, log=log,
                            block_size=block_size, num_pages=None if pages is None else int(pages),
                            max_live=int(geometry.get("max_live", args.max_live)),
                            fixed_products=not args.timed_products)  # fmt: skip
            log("ready")
            if "step" not in record:
                continue
        step = record["step"]
        logits = replay.step(record.get("entries", []), record.get("end", []))
        if logits is not None:
            logits.contiguous().numpy().astype("<f4", copy=False).tofile(os.path.join(args.out, f"{step}.f32"))
        print(f"done {step}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())

"""Trace replay: feed given token ids through the model step by step and write logits.

It samples nothing and has no forward pass, cache or loader of its own: it loads the
model as the engine does, takes pages from the engine's cache manager and calls the
engine's step function (`ModelRunner.step`), so what it measures is what generation
runs.  The reference's nearest pieces are `ModelRunner.run` for tools and the
`full_logits` fixture (atomserve/runner.py:182-192, tests/conftest.py:79-98).

Input, one JSON object per line on standard input:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

`entries` are one batch: each request's next tokens and the places among them whose
logits are wanted.  `end` lists requests finished after the step; their pages return
to the pool.  For a step with wanted places `<out>/<step>.f32` receives the logits as
little-endian float32 [wanted, vocab], in the order of the entries and of `want`.
After every step `done <step>` is printed and flushed.
"""

import argparse
import json
import os
import sys

DTYPES = {"bfloat16": "bfloat16", "bf16": "bfloat16", "float32": "float32", "fp32": "float32"}
BLOCK_SIZE = 16
MAX_LIVE = 8


class Replay:
    def __init__(self, model_dir: str, dtype: str, max_tokens: int, device: str = "cuda:0", log=None):
        import torch

        from atomserve_amd.cache.manager import CacheManager
        from atomserve_amd.engine.runner import ModelRunner
        from atomserve_amd.weights.loader import load_model

        self.log = log or (lambda msg: None)
        torch_dtype = getattr(torch, DTYPES[dtype])
        self.log(f"loading {model_dir} ({DTYPES[dtype]}) ...")
        self.model, self.arch, self.config = load_model(model_dir, torch_dtype, device)
        num_blocks = max(1, -(-max_tokens // BLOCK_SIZE))
        self.manager = CacheManager(self.model.cache_requests(), BLOCK_SIZE, num_blocks, MAX_LIVE)
        self.runner = ModelRunner(self.model, self.manager)
        self.live: dict = {}  # request id -> [RequestCache, tokens computed so far]

    def step(self, entries: list, end: list):
        """Run one step; returns the logits of its wanted places as a CPU tensor, or None."""
        from atomserve_amd.engine.batch import Row

        rows = []
        seen = set()
        for e in entries:
            rid, tokens, want = e["id"], [int(t) for t in e["tokens"]], [int(w) for w in e.get("want", [])]
            if rid in seen:
                raise ValueError(f"request {rid!r} appears twice in one step")
            seen.add(rid)
            if not tokens:  # an entry that brings nothing runs nothing
                if want:
                    raise ValueError(f"request {rid!r} wants logits of a step in which it has no tokens")
                continue
            if rid not in self.live:
                self.live[rid] = [self.manager.new_request(), 0]
            rc, computed = self.live[rid]
            if not self.manager.reserve(rc, computed, len(tokens)):
                raise RuntimeError(
                    f"the cache pool ({self.manager.num_blocks} pages of {BLOCK_SIZE} tokens) has no room for "
                    f"request {rid!r}; --max-tokens is too small for the live requests"
                )
            rows.append(Row(tokens, computed, rc.tables, want, rc.state_slot))
        logits = None
        if rows:
            out = self.runner.step(rows)
            if out.shape[0]:
                logits = out.cpu()
            for e in entries:
                if e["tokens"]:
                    state = self.live[e["id"]]
                    state[1] += len(e["tokens"])
                    self.manager.release_behind_window(state[0], state[1])
        for rid in end:
            if rid in self.live:
                self.manager.release(self.live.pop(rid)[0])
        return logits


def build_parser() -> argparse.ArgumentParser:
    p = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    p.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    p.add_argument("--dtype", required=True, choices=sorted(DTYPES), help="bfloat16: what serving uses; float32: true 32-bit")
    p.add_argument("--out", required=True, help="folder for <step>.f32 files")
    p.add_argument("--max-tokens", type=int, required=True, help="most tokens that live requests hold at any time")
    p.add_argument("--device", default="cuda:0", help=argparse.SUPPRESS)
    return p


def main(argv=None, stdin=None) -> int:
    args = build_parser().parse_args(argv)
    stdin = stdin or sys.stdin

    def log(msg):
        print(f"trace_run: {msg}", file=sys.stderr, flush=True)

    os.makedirs(args.out, exist_ok=True)
    replay = Replay(args.model, args.dtype, args.max_tokens, device=args.device, log=log)
    log("ready")
    for line in stdin:
        line = line.strip()
        if not line:
            continue
        record = json.loads(line)
        step = record["step"]
        logits = replay.step(record.get("entries", []), record.get("end", []))
        if logits is not None:
            logits.contiguous().numpy().astype("<f4", copy=False).tofile(os.path.join(args.out, f"{step}.f32"))
        print(f"done {step}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())

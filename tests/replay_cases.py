"""Traces for the replay tool, and their comparison with the plain implementation.

A trace is a list of steps {"step", "entries": [{"id", "tokens", "want"}], "end"}; the
same requests are cut in different ways, and every wanted row of logits is compared
with the plain implementation's logits of the whole sequence at that position."""

import random

import torch

from tests import plain_qwen3 as plain


def whole(rid, ids):
    return [{"step": 0, "entries": [{"id": rid, "tokens": list(ids), "want": list(range(len(ids)))}], "end": [rid]}]


def prefill_then_decode(rid, ids, tail=32):
    head = len(ids) - tail
    steps = [{"step": 0, "entries": [{"id": rid, "tokens": list(ids[:head]), "want": [head - 1]}], "end": []}]
    for i in range(head, len(ids)):
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": [ids[i]], "want": [0]}],
                      "end": [rid] if i == len(ids) - 1 else []})  # fmt: skip
    return steps


def portions(rid, ids, sizes=(9, 2, 17, 3, 2, 31, 8, 5, 64, 2, 11)):
    steps, at, i = [], 0, 0
    while at < len(ids):
        n = min(sizes[i % len(sizes)], len(ids) - at)
        if len(ids) - at - n == 1:  # never leave a single token: portions go down to two
            n += 1
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": list(ids[at : at + n]),
                                                       "want": list(range(n))}], "end": []})  # fmt: skip
        at += n
        i += 1
    steps[-1]["end"] = [rid]
    return steps


def mixed(requests: dict, seed=0, max_live=4, prompt_fraction=0.6, sizes=(2, 7, 19, 3, 33, 12), prompt_lengths=None):
    """Up to `max_live` requests at a time: portions of some prompts beside single tokens of
    others; a request's turn may be skipped; new ones start as old ones end.
    prompt_lengths: request id -> how many of its tokens come in portions (default: a fraction)."""
    rng = random.Random(seed)
    waiting = list(requests.items())
    live, steps = {}, []
    while waiting or live:
        while waiting and len(live) < max_live:
            rid, ids = waiting.pop(0)
            prompt = (prompt_lengths or {}).get(rid, int(len(ids) * prompt_fraction))
            live[rid] = {"ids": ids, "at": 0, "prompt": max(2, prompt)}
        entries, end = [], []
        for rid, st in list(live.items()):
            if len(live) > 1 and rng.random() < 0.15:
                continue  # left out of this step; goes on later
            left = len(st["ids"]) - st["at"]
            if st["at"] < st["prompt"]:
                n = min(rng.choice(sizes), st["prompt"] - st["at"])
                if st["prompt"] - st["at"] - n == 1:
                    n += 1
            else:
                n = 1
            n = min(n, left)
            tokens = st["ids"][st["at"] : st["at"] + n]
            want = list(range(n)) if rng.random() < 0.5 or n == 1 else [n - 1]
            entries.append({"id": rid, "tokens": list(tokens), "want": want})
            st["at"] += n
            if st["at"] == len(st["ids"]):
                end.append(rid)
                del live[rid]
        if entries:
            steps.append({"step": len(steps), "entries": entries, "end": end})
    return steps


def live_token_bound(steps, unit=64):
    """Most tokens that live requests hold at any time, each rounded up to `unit`."""
    held, worst = {}, 0
    for s in steps:
        for e in s["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        worst = max(worst, sum(-(-n // unit) * unit for n in held.values()))
        for rid in s["end"]:
            held.pop(rid, None)
    return worst


class Spread:
    """Largest and root-mean-square of the differences added to it."""

    def __init__(self):
        self.worst, self.sum_sq, self.count = 0.0, 0.0, 0

    def add(self, diff):
        self.worst = max(self.worst, float(diff.abs().max()))
        self.sum_sq += float(diff.double().pow(2).sum())
        self.count += diff.numel()

    @property
    def rms(self):
        return (self.sum_sq / max(1, self.count)) ** 0.5


class Comparison:
    """What a trace's wanted rows are against the plain model: `err` engine - plain; `noise` the plain
    model with its activations rounded to bfloat16 - plain (filled when asked for); `scale` the largest
    |logit| of the plain model; `rows` compared.  Unpacks as (largest |difference|, scale, rows)."""

    def __init__(self):
        self.err, self.noise, self.scale, self.rows = Spread(), Spread(), 0.0, 0

    def __iter__(self):
        return iter((self.err.worst, self.scale, self.rows))


# 32-bit: the engine and the float64 plain model differ by float32 rounding, a few 1e-6 of the largest logit.
TOL_FLOAT32 = 2e-5
# bfloat16: the engine may be as far from the exact logits as the plain model itself moves when its
# activations are rounded to bfloat16 at the places where an engine that stores them so must round them
# (tests/plain_qwen3.py `storage`), times these factors: root mean square over every compared logit, and
# the largest single difference (the extreme of thousands of draws: it scatters more).  Over the 143
# comparisons of tests/test_model_gpu.py the engine came to 1.09 and 1.33 of the plain model's own noise
# at most; a fault of the cache or a kernel moves logits by their own size, tens of times the noise.
BF16_RMS_FACTOR, BF16_WORST_FACTOR = 1.25, 2.0


def within_bounds(result: Comparison, dtype: str, tol32: float = TOL_FLOAT32) -> None:
    if dtype == "float32":
        assert result.err.worst <= tol32 * max(result.scale, 1.0), \
            f"float32: |difference| {result.err.worst:.3e} against |logits| {result.scale:.3e}"  # fmt: skip
        return
    assert result.noise.count == result.err.count and result.noise.count > 0, "the rounding noise was not measured"
    assert result.err.rms <= BF16_RMS_FACTOR * result.noise.rms and result.err.worst <= BF16_WORST_FACTOR * result.noise.worst, (
        f"bfloat16: engine - plain rms {result.err.rms:.3e} max {result.err.worst:.3e}; "
        f"rounding alone moves the plain model by rms {result.noise.rms:.3e} max {result.noise.worst:.3e}")  # fmt: skip


def plain_rows(raw, weights, ids, cache: dict, key, rounded: bool, plain_kwargs=None):
    """The plain model's logits of a whole sequence (cached under `key`): exact, or with bfloat16 activations."""
    key = (key, "rounded") if rounded else key
    if key not in cache:
        kwargs = dict(plain_kwargs or {})
        if rounded:
            kwargs.update(batched=True, storage=torch.bfloat16)
        cache[key] = plain.logits(raw, weights, ids, **kwargs).float().cpu()
    return cache[key]


def run_and_compare(replay, steps, requests: dict, raw, weights, reference_cache: dict, plain_kwargs=None, noise=False):
    """Feed `steps` to a `Replay` and compare every wanted row with the plain model's logits of the whole
    sequence at that place; returns a `Comparison`.
    plain_kwargs: how the plain model runs (default: float64 on the CPU, the loop form).
    noise: also measure what rounding to bfloat16 alone does to the plain model at the same rows."""
    at = {rid: 0 for rid in requests}
    result = Comparison()
    for s in steps:
        logits = replay.step(s["entries"], s["end"])
        k = 0
        for e in s["entries"]:
            rid = e["id"]
            ref = plain_rows(raw, weights, requests[rid], reference_cache, rid, False, plain_kwargs)
            for w in e["want"]:
                want = ref[at[rid] + w]
                result.err.add(logits[k] - want)
                if noise:
                    result.noise.add(plain_rows(raw, weights, requests[rid], reference_cache, rid, True, plain_kwargs)[at[rid] + w] - want)
                result.scale = max(result.scale, float(want.abs().max()))
                k += 1
                result.rows += 1
            at[rid] += len(e["tokens"])
        assert (logits is None and k == 0) or logits.shape[0] == k
    return result


def random_ids(vocab, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()

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


def run_and_compare(replay, steps, requests: dict, raw, weights, reference_cache: dict, plain_kwargs=None):
    """Feed `steps` to a `Replay`; returns (largest |difference|, largest |reference|, rows compared).
    plain_kwargs: how the plain model runs (default: float64 on the CPU, the loop form)."""
    at = {rid: 0 for rid in requests}
    worst, scale, rows = 0.0, 0.0, 0
    for s in steps:
        logits = replay.step(s["entries"], s["end"])
        k = 0
        for e in s["entries"]:
            rid = e["id"]
            if rid not in reference_cache:
                reference_cache[rid] = plain.logits(raw, weights, requests[rid], **(plain_kwargs or {})).float().cpu()
            ref = reference_cache[rid]
            for w in e["want"]:
                got = logits[k]
                want = ref[at[rid] + w]
                worst = max(worst, float((got - want).abs().max()))
                scale = max(scale, float(want.abs().max()))
                k += 1
                rows += 1
            at[rid] += len(e["tokens"])
        assert (logits is None and k == 0) or logits.shape[0] == k
    return worst, scale, rows


def random_ids(vocab, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()

"""Turns next-token logits into chosen tokens, for a whole batch at once, on the GPU
(reference atomserve/sampler.py:1-168).

    logits -> presence penalty -> top-k -> / temperature -> softmax -> top-p -> draw

Every row has its own settings.  A batch that is all greedy is one argmax kernel;
otherwise one sampling kernel handles every row, greedy ones included.  The noise of
the draw is a function of (the request's seed, how many tokens it has sampled, the
candidate), so a request's stream does not depend on its batch neighbours; requests
without a seed get one drawn by the engine when they are submitted.
"""

import numpy as np
import torch

from atomserve_amd.kernels import ops


class Sampler:
    def __init__(self, device):
        self.device = torch.device(device)

    def release(self, seq_id: int) -> None:
        """Nothing is kept per request: the random stream is a function of the request's own
        seed and token count (the reference keeps a generator here, sampler.py:58-60)."""

    def sample(self, logits: torch.Tensor, seqs) -> list:
        """logits [B, vocab] fp32, row i belongs to seqs[i]; returns B token ids (one host
        synchronisation, the step's only one)."""
        out = self.launch(logits, seqs)
        return [] if out is None else out.tolist()

    def launch(self, logits: torch.Tensor, seqs, ahead: int = 0):
        """The same without waiting: the B token ids as an int32 tensor on the GPU (None for no rows).
        ahead: how many tokens each sequence will have sampled by then beyond what it holds now (a step
        put on the GPU before the one before it was read)."""
        if not seqs:
            return None
        B, vocab = logits.shape
        if B != len(seqs):
            raise ValueError(f"{B} rows of logits for {len(seqs)} sequences")
        params = [s.params for s in seqs]
        logits = self._apply_presence_penalty(logits, seqs)
        out = torch.empty(B, dtype=torch.int32, device=self.device)
        if all(p.temperature == 0 for p in params):
            ops.argmax(logits, out)
            return out
        top_k, kept = [], []
        for p in params:
            k = p.top_k if 0 < p.top_k < vocab else 0
            top_k.append(k)
            # candidates the row keeps; all tokens (k == 0) and more than the kernels rank in LDS
            # are left to the one-workgroup kernel
            kept.append(1 if p.temperature <= 0 or p.top_p <= 0 else (k or ops.SAMPLE_MAX_TOP_K + 1))
        # One upload: int32 rows (temperature and top_p as their bit patterns, top_k, tokens sampled
        # so far), then the 64-bit seeds.
        host = np.empty(6 * B, dtype=np.int32)
        host[0:B].view(np.float32)[:] = [max(p.temperature, 0.0) for p in params]
        host[B : 2 * B].view(np.float32)[:] = [p.top_p for p in params]
        host[2 * B : 3 * B] = top_k
        host[3 * B : 4 * B] = [s.num_output_tokens + ahead for s in seqs]
        host[4 * B :].view(np.int64)[:] = [_as_int64(s.noise_seed) for s in seqs]
        dev = torch.from_numpy(host).to(self.device, non_blocking=True)
        floats, ints = dev[: 2 * B].view(torch.float32), dev[2 * B : 4 * B]
        ops.sample(logits, floats[:B], ints[:B], floats[B:], dev[4 * B :].view(torch.int64), ints[B:], out,
                   max_top_k=max(kept))  # fmt: skip
        return out

    def _apply_presence_penalty(self, logits, seqs):
        """logits with each penalised row's amount taken off every token the row's request has
        generated so far, each token once however often it came (reference atomserve/sampler.py:144-168).
        The rows are copied first: the caller's logits stay as the model made them."""
        marks = []  # per penalised row: (row, its distinct generated tokens, amount)
        for row, seq in enumerate(seqs):
            amount = seq.params.presence_penalty
            if amount != 0 and seq.num_output_tokens:
                marks.append((row, np.unique(np.asarray(seq.output_ids, dtype=np.int32)), amount))
        if not marks:
            return logits
        total = sum(len(tokens) for _, tokens, _ in marks)
        # one upload: [rows | tokens | amounts as bit patterns]
        host = np.empty(3 * total, dtype=np.int32)
        at = 0
        for row, tokens, amount in marks:
            n = len(tokens)
            host[at : at + n] = row
            host[total + at : total + at + n] = tokens
            host[2 * total + at : 2 * total + at + n].view(np.float32)[:] = amount
            at += n
        dev = torch.from_numpy(host).to(self.device, non_blocking=True)
        logits = logits.clone()
        ops.apply_penalty(logits, dev[:total], dev[total : 2 * total], dev[2 * total :].view(torch.float32))
        return logits


def _as_int64(seed: int) -> int:
    seed &= (1 << 64) - 1
    return seed - (1 << 64) if seed >= (1 << 63) else seed

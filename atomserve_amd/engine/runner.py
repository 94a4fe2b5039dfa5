"""The step function: "run these tokens of these requests" as one pass over the GPU
(reference atomserve/runner.py:59-212).

`ModelRunner.step(rows)` runs exactly the tokens it is given, as one batch, from the
cache that earlier steps left, writes their keys and values, and returns the logits at
the wanted places.  It never changes a sequence: advancing and appending is the
scheduler's work, so the same plan can be inspected or retried.
"""

import torch

from atomserve_amd.cache.manager import CacheManager
from atomserve_amd.cache.pools import CachePools
from atomserve_amd.engine.batch import Row, Staging, StepBatch
from atomserve_amd.engine.sequence import StepResult
from atomserve_amd.sampling.sampler import Sampler


def rows_for(seqs, num_new_tokens) -> list:
    """The usual rows: each sequence's next uncomputed tokens, logits at its last token only
    if that is its last known token (reference atomserve/runner.py:59-68)."""
    rows = []
    for seq, n in zip(seqs, num_new_tokens, strict=True):
        start = seq.num_computed_tokens
        if n < 1 or start + n > seq.num_tokens:
            raise ValueError(f"cannot run tokens {start}:{start + n} of {seq.num_tokens}")
        want = [n - 1] if seq.reaches_end(n) else []
        rows.append(Row(seq.token_ids[start : start + n], start, seq.cache.tables, want, seq.cache.state_slot))
    return rows


class ModelRunner:
    """Owns the model, the cache pools and the sampler; executes one step for a list of rows."""

    def __init__(self, model, manager: CacheManager, pools: CachePools = None):
        self.model = model
        self.manager = manager
        self.device = model.env.device
        self.pools = pools if pools is not None else CachePools(manager, model.env.dtype, self.device)
        self.sampler = Sampler(self.device)
        self.staging = Staging(self.device)
        self.vocab_size = model.plan.vocab_size

    def prepare(self, rows) -> StepBatch:
        return StepBatch(rows, self.manager.block_size, len(self.manager.paged_groups), self.vocab_size,
                         self.device, pools=self.pools, staging=self.staging)  # fmt: skip

    @torch.inference_mode()
    def step(self, rows) -> torch.Tensor:
        """Logits [sum of len(row.want), vocab] fp32, in the order of the rows and of `want`."""
        batch = self.prepare(rows)
        return self.model.forward(batch)

    @torch.inference_mode()
    def run(self, seqs, num_new_tokens) -> torch.Tensor:
        """One step for sequences; row j of the result belongs to the j-th sequence that
        reaches its end this step (reference atomserve/runner.py:182-192)."""
        return self.step(rows_for(seqs, num_new_tokens))

    @torch.inference_mode()
    def execute(self, out) -> list:
        """Run one scheduled step and sample: a sequence that reaches the end of its known
        tokens gets one new token (reference atomserve/runner.py:194-212)."""
        logits = self.step(rows_for(out.seqs, out.num_new_tokens))
        sampling = [s for s, n in zip(out.seqs, out.num_new_tokens, strict=True) if s.reaches_end(n)]
        sampled = iter(self.sampler.sample(logits, sampling))
        return [
            StepResult(tokens=[next(sampled)] if seq.reaches_end(n) else [], num_computed=seq.num_computed_tokens + n)
            for seq, n in zip(out.seqs, out.num_new_tokens, strict=True)
        ]

"""Dense gated feed-forward: down( act(gate(x)) * up(x) ) with gate and up stacked into
one matrix (reference atomserve/model.py:339-360)."""

import torch

from atomserve_amd.kernels import ops
from atomserve_amd.parts.base import FeedForward, PendingNorm, SplitSums, WeightDecl, register


class GatedMLP(FeedForward):
    capturable = True
    takes_pending_norm = True
    adds_to_residual = True

    def __init__(self, spec, env):
        super().__init__(spec, env)
        if spec.activation != "silu":
            raise ValueError(f"activation {spec.activation!r} has no kernel (only 'silu')")

    def weight_decls(self) -> dict:
        s = self.spec
        return {
            "gate_up.weight": WeightDecl((2 * s.intermediate_size, s.hidden_size)),
            "down.weight": WeightDecl((s.hidden_size, s.intermediate_size)),
        }

    def bind(self, tensors: dict) -> None:
        super().bind(tensors)
        # what the products of a decode step stream: the matrices with their copies in wave order
        self.gate_up = ops.Streamed(self.gate_up_weight, self.env.stream_copies)
        self.down = ops.Streamed(self.down_weight, self.env.stream_copies)

    def streamed(self) -> list:
        return [self.gate_up, self.down]

    def forward(self, h, step, residual=None, next_norm=None):
        s, env = self.spec, self.env
        pending = isinstance(h, PendingNorm)
        T, device = (h.x.shape[0], h.x.device) if pending else (h.shape[0], h.device)
        act = torch.empty((T, s.intermediate_size), dtype=env.dtype, device=device)
        if not (pending and h.gemm_gated(self.gate_up, act, s.activation)):
            ops.gemm_silu_mul(h.rows() if pending else h, self.gate_up, act, env.products)
        if residual is not None and next_norm is not None:
            link = next_norm.absorb(act, self.down, residual)
            if link is not None:
                return link
            if next_norm.takes_split_sums:
                plan = ops.gemm_split_plan(T, s.hidden_size, act.shape[1], env.dtype)
                if plan is not None:
                    return SplitSums(ops.gemm_split(act, self.down, plan))
        y = torch.empty((T, s.hidden_size), dtype=env.dtype, device=device)
        ops.gemm(act, self.down, y, env.products)
        return y


register("feed_forward", "gated_mlp", GatedMLP)

"""RMSNorm: weight * x / sqrt(mean(x^2) + eps), accumulated in fp32 and rounded once
(reference atomserve/model.py:125-139).  The residual sum that precedes a norm in a
pre-norm layer is fused into the same kernel: the fp32 residual stream `x` receives
`delta` and the normalised result is written in the compute dtype."""

import torch

from atomserve_amd.kernels import ops
from atomserve_amd.parts.base import Norm, PendingNorm, SplitSums, WeightDecl, register


class PendingRMSNorm(PendingNorm):
    """x * gain (rounded to the compute dtype) and the sums of x^2 per 16 columns: a product of
    `scaled` times 1 / rms is the product of the normalised rows."""

    def __init__(self, norm, x, scaled, ssq):
        super().__init__(norm, x)
        self.scaled, self.ssq = scaled, ssq

    def gemm(self, w, out) -> None:
        ops.gemm_scaled(self.scaled, self.ssq, self.norm.spec.eps, w, out)

    def gemm_gated(self, w, out, activation) -> bool:
        if activation != "silu":
            return False
        ops.gemm_scaled(self.scaled, self.ssq, self.norm.spec.eps, w, out, gated=True)
        return True


class RMSNorm(Norm):
    capturable = True
    takes_split_sums = True

    def weight_decls(self) -> dict:
        return {"weight": WeightDecl((self.spec.size,), role="vector")}

    def bind(self, tensors: dict) -> None:
        super().bind(tensors)
        self.gain_f32 = self.weight.float()  # what the fused product reads (exact: bf16 widens)

    def absorb(self, a, w, x):
        M, N = x.shape
        if not ops.gemm_link_supported(M, N, a.shape[1], self.env.dtype, w):
            return None
        scaled = torch.empty((M, N), dtype=self.env.dtype, device=x.device)
        ssq = torch.empty((M, -(-N // 16)), dtype=torch.float32, device=x.device)
        ops.gemm_link(a, w, x, self.gain_f32, scaled, ssq)
        return PendingRMSNorm(self, x, scaled, ssq)

    def forward(self, x, delta=None, rows=None, update_residual=True) -> torch.Tensor:
        """x: fp32 [T, size] residual stream.  delta: pending sum in the compute dtype (or as the
        partial sums of the product that makes it, `SplitSums`), or None.
        rows: int32 row selection, or None for all rows.  Returns [rows, size], compute dtype."""
        n_out = x.shape[0] if rows is None else rows.shape[0]
        out = torch.empty((n_out, self.spec.size), dtype=self.env.dtype, device=x.device)
        if isinstance(delta, SplitSums):
            ops.rmsnorm(x, self.weight, self.spec.eps, out, rows=rows, update_x=update_residual, split_sums=delta.sums)
        else:
            ops.rmsnorm(x, self.weight, self.spec.eps, out, delta=delta, rows=rows, update_x=update_residual)
        return out


register("norm", "rmsnorm", RMSNorm)

"""RMSNorm: weight * x / sqrt(mean(x^2) + eps), accumulated in fp32 and rounded once
(reference atomserve/model.py:125-139).  The residual sum that precedes a norm in a
pre-norm layer is fused into the same kernel: the fp32 residual stream `x` receives
`delta` and the normalised result is written in the compute dtype."""

import torch

from atomserve_amd.kernels import ops
from atomserve_amd.parts.base import Norm, WeightDecl, register


class RMSNorm(Norm):
    def weight_decls(self) -> dict:
        return {"weight": WeightDecl((self.spec.size,), role="vector")}

    def forward(self, x, delta=None, rows=None, update_residual=True) -> torch.Tensor:
        """x: fp32 [T, size] residual stream.  delta: pending sum in the compute dtype, or None.
        rows: int32 row selection, or None for all rows.  Returns [rows, size], compute dtype."""
        n_out = x.shape[0] if rows is None else rows.shape[0]
        out = torch.empty((n_out, self.spec.size), dtype=self.env.dtype, device=x.device)
        ops.rmsnorm(x, self.weight, self.spec.eps, out, delta=delta, rows=rows, update_x=update_residual)
        return out


register("norm", "rmsnorm", RMSNorm)

"""Rotary position encoding, "rotate-half" layout: the pair (x[i], x[i + R/2]) turns
by position * theta^(-2i/R) (reference atomserve/model.py:142-185).

The part owns the frequencies and, once per step, the table of (cos, sin) of every
token's angles, which every layer with the same spec then shares.  The angles are
formed and range-reduced in fp64 on the device, so that positions in the tens of
thousands lose nothing; the rotation that uses them is fp32.
"""

import torch

from atomserve_amd.kernels import ops
from atomserve_amd.parts.base import Position, register


class RotaryHalf(Position):
    capturable = True
    pairs = "half"

    def __init__(self, spec, env):
        super().__init__(spec, env)
        if spec.rotary_dim % 2 or spec.rotary_dim <= 0:
            raise ValueError(f"rotary_dim {spec.rotary_dim} must be positive and even")
        i = torch.arange(0, spec.rotary_dim, 2, dtype=torch.float64)
        self.inv_freq = (1.0 / (float(spec.theta) ** (i / spec.rotary_dim))).to(env.device)

    def prepare(self, step) -> torch.Tensor:
        """cos/sin of this step's tokens, fp32 [T, R/2, 2]; computed once per step and spec."""
        key = ("rope_half", self.spec.rotary_dim, self.spec.theta)
        table = step.shared.get(key)
        if table is None:
            table = torch.empty((step.num_tokens, self.spec.rotary_dim // 2, 2), dtype=torch.float32,
                                device=self.env.device)  # fmt: skip
            ops.rope_table(step.positions, self.inv_freq, table)
            step.shared[key] = table
        return table


register("position", "rope_half", RotaryHalf)

"""Arrangements: how one layer orders its norms, mixer, feed-forward and residual sums.

"prenorm":  x += mixer(norm(x));  x += ffn(norm(x))   (reference atomserve/model.py:378-382)

The residual stream `x` is fp32 in both precisions.  A part's output is not added at
once: it travels as the pending `delta` to the next norm, whose kernel adds it into
`x` and normalises in one pass.  With few rows (decoding) both steps move into the matrix
products around them instead: a part's last product adds into `x` and leaves the next norm
pending (`Norm.absorb`), and the next part's first product finishes it (`PendingNorm`).
"""

from atomserve_amd.parts.base import Arrangement, PendingNorm, build, register


class PreNormBlock(Arrangement):
    def __init__(self, spec, env):
        super().__init__(spec, env)
        self.mixer_norm = build("norm", spec.mixer_norm, env)
        self.mixer = build("mixer", spec.mixer, env)
        self.ffn_norm = build("norm", spec.ffn_norm, env)
        self.ffn = build("feed_forward", spec.ffn, env)

    def parts(self) -> dict:
        return {"mixer_norm": self.mixer_norm, "mixer": self.mixer, "ffn_norm": self.ffn_norm, "ffn": self.ffn}

    def first_norm(self):
        return self.mixer_norm

    def forward(self, x, delta, step, cache, next_norm=None):
        delta = self.apply(self.mixer_norm, self.mixer, self.ffn_norm, x, delta, step, cache)
        return self.apply(self.ffn_norm, self.ffn, next_norm, x, delta, step)

    @staticmethod
    def apply(norm, part, next_norm, x, delta, *args):
        """part(norm(x + delta)): the part's output still to be added, or the PendingNorm of
        `next_norm` if the part added it itself.  `delta` may be the PendingNorm of `norm`."""
        if isinstance(delta, PendingNorm):
            h = delta if part.takes_pending_norm else delta.rows()
        else:
            h = norm.forward(x, delta)
        if part.adds_to_residual:
            return part.forward(h, *args, residual=x, next_norm=next_norm)
        return part.forward(h, *args)


register("arrangement", "prenorm", PreNormBlock)

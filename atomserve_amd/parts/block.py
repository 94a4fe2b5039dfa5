"""Arrangements: how one layer orders its norms, mixer, feed-forward and residual sums.

"prenorm":  x += mixer(norm(x));  x += ffn(norm(x))   (reference atomserve/model.py:378-382)

The residual stream `x` is fp32 in both precisions.  A part's output is not added at
once: it travels as the pending `delta` to the next norm, whose kernel adds it into
`x` and normalises in one pass.
"""

from atomserve_amd.parts.base import Arrangement, build, register


class PreNormBlock(Arrangement):
    def __init__(self, spec, env):
        super().__init__(spec, env)
        self.mixer_norm = build("norm", spec.mixer_norm, env)
        self.mixer = build("mixer", spec.mixer, env)
        self.ffn_norm = build("norm", spec.ffn_norm, env)
        self.ffn = build("feed_forward", spec.ffn, env)

    def parts(self) -> dict:
        return {"mixer_norm": self.mixer_norm, "mixer": self.mixer, "ffn_norm": self.ffn_norm, "ffn": self.ffn}

    def forward(self, x, delta, step, cache):
        h = self.mixer_norm.forward(x, delta)
        delta = self.mixer.forward(h, step, cache)
        h = self.ffn_norm.forward(x, delta)
        return self.ffn.forward(h, step)


register("arrangement", "prenorm", PreNormBlock)

"""Arrangements: how a block wires its norms, its mixer and its feed-forward."""
from __future__ import annotations

from .base import ARRANGEMENTS, Arrangement


@ARRANGEMENTS.register("prenorm_residual")
class PreNormResidual(Arrangement):
    """x = x + mixer(norm_a(x)); x = x + feed_forward(norm_f(x))   (reference main_models_new.py:146-152)."""
    part_names = ("mixer_norm", "mixer", "feed_forward_norm", "feed_forward")

    def __init__(self, layer_spec, tensors, ops):
        super().__init__(layer_spec, tensors, ops)
        self.mixer_norm, self.mixer = self.parts["mixer_norm"], self.parts["mixer"]
        self.ffn_norm, self.ffn = self.parts["feed_forward_norm"], self.parts["feed_forward"]

    def forward(self, x, ctx):
        # the stream `x` is replaced by each sub-layer's result, so the residual passed down is spent and a part may
        # write its result over it; whether the block's own input is spent too, the caller says in ctx
        mctx = ctx.of("mixer")
        if getattr(self.mixer, "fuses_norm", False):
            x = self.mixer.forward(x, mctx, residual=x, norm=self.mixer_norm)
        else:
            x = self.mixer.forward(self.mixer_norm(x), mctx, residual=x)
        if getattr(self.ffn, "fuses_norm", False):
            return self.ffn.forward(x, residual=x, norm=self.ffn_norm, residual_is_spent=True)
        return self.ffn.forward(self.ffn_norm(x), residual=x)

"""Arrangements: how a block wires its norms, its mixer and its feed-forward."""
from __future__ import annotations

from .base import ARRANGEMENTS, build_part


@ARRANGEMENTS.register("prenorm_residual")
class PreNormResidual:
    """x = x + mixer(norm_a(x)); x = x + feed_forward(norm_f(x))   (reference main_models_new.py:146-152)."""

    def __init__(self, layer_spec, tensors, ops):
        self.mixer_norm = build_part(layer_spec.mixer_norm, tensors, ops)
        self.mixer = build_part(layer_spec.mixer, tensors, ops)
        self.ffn_norm = build_part(layer_spec.feed_forward_norm, tensors, ops)
        self.ffn = build_part(layer_spec.feed_forward, tensors, ops)

    def forward(self, x, ctx):
        # the stream `x` is replaced by each sub-layer's result, so the residual passed down is spent and a part may
        # write its result over it; whether the block's own input is spent too, the caller says in ctx
        if getattr(self.mixer, "fuses_norm", False):
            x = self.mixer.forward(x, ctx, residual=x, norm=self.mixer_norm)
        else:
            x = self.mixer.forward(self.mixer_norm(x), ctx, residual=x)
        if getattr(self.ffn, "fuses_norm", False):
            return self.ffn.forward(x, residual=x, norm=self.ffn_norm, residual_is_spent=True)
        return self.ffn.forward(self.ffn_norm(x), residual=x)

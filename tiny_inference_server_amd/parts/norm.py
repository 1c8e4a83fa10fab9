"""Norm parts."""
from __future__ import annotations

from .base import NORMS, to_gain


@NORMS.register("rmsnorm_l2")
class RmsNormL2:
    """y = x * sqrt(D) / (||x||_2 + eps) * gain, computed in 32-bit.

    The reference's norm (main_models_new.py:31-42): the L2 norm of the row with eps added to the norm
    itself, not under the root. params: width, eps. tensors: gain (width,).
    """
    graph_safe = True

    @classmethod
    def tensor_shapes(cls, params):
        return {"gain": (params["width"],)}

    def __init__(self, spec, tensors, ops):
        self.ops = ops
        self.width = int(spec.params["width"])
        self.eps = float(spec.params["eps"])
        self.gain = to_gain(ops, tensors.of(spec, "gain"))

    def as_rms(self):
        """(gain, eps) for kernels that fuse this norm into what follows it."""
        return self.gain, self.eps

    def __call__(self, x, out=None):
        return self.ops.rmsnorm(x, self.gain, self.eps, out=out)

"""Feed-forward parts."""
from __future__ import annotations

import torch

from .base import FEED_FORWARDS, to_compute


@FEED_FORWARDS.register("swiglu")
class SwiGlu:
    """y = (silu(x.W1) * (x.W2)) . Wfc (+ residual), dense (reference main_models_new.py:44-60).

    params: d_model, hidden. tensors: gate (d_model, hidden), up (d_model, hidden), down (hidden, d_model),
    stored [in, out].
    """
    graph_safe = True

    @classmethod
    def tensor_shapes(cls, params):
        d, f = params["d_model"], params["hidden"]
        return {"gate": (d, f), "up": (d, f), "down": (f, d)}

    def __init__(self, spec, tensors, ops):
        self.ops = ops
        # one projection for gate and up: rows of the [out, in] matrix alternate gate_0, up_0, gate_1, up_1, ...
        # so that the gating can be done where the product's results still sit in registers
        gate, up = tensors.of(spec, "gate"), tensors.of(spec, "up")
        self.w_gate_up = to_compute(ops, torch.stack((gate.t(), up.t()), dim=1).reshape(2 * gate.shape[1], gate.shape[0]))
        self.w_down = to_compute(ops, tensors.of(spec, "down").t())

    fuses_norm = True

    def forward(self, x, residual=None, norm=None, residual_is_spent=False):
        ops = self.ops
        if norm is not None and not hasattr(norm, "as_rms"):
            x, norm = norm(x), None
        hidden = ops.linear_swiglu(x, self.w_gate_up, rms=norm.as_rms() if norm is not None else None)
        return ops.linear(hidden, self.w_down, residual=residual, reuse_residual=residual_is_spent)

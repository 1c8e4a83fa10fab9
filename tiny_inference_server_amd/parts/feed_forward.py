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
        # one projection for gate and up: rows [0, hidden) of the [out, in] matrix are the gate
        self.w_gate_up = to_compute(ops, torch.cat((tensors.of(spec, "gate"), tensors.of(spec, "up")), dim=1).t())
        self.w_down = to_compute(ops, tensors.of(spec, "down").t())

    def forward(self, x, residual=None):
        ops = self.ops
        return ops.linear(ops.swiglu(ops.linear(x, self.w_gate_up)), self.w_down, residual=residual)

"""Position encoding parts."""
from __future__ import annotations

import torch

from .base import POSITION_ENCODINGS


@POSITION_ENCODINGS.register("rotary")
class Rotary:
    """Rotary encoding of queries and keys.

    theta_j = base^(-2j/head_dim); the angle at position p is p * theta_j in 32-bit (reference
    main_models_new.py:63-69). pairing "half" rotates (j, j + head_dim/2) (main_models_new.py:71-80),
    "interleaved" rotates (2j, 2j+1). params: head_dim, base, max_context, pairing.
    """

    @classmethod
    def tensor_shapes(cls, params):
        return {}

    def __init__(self, spec, tensors, ops):
        p = spec.params
        self.head_dim = int(p["head_dim"])
        self.max_context = int(p["max_context"])
        pairing = p.get("pairing", "half")
        if pairing not in ("half", "interleaved"):
            raise ValueError(f"rotary pairing {pairing!r}: use 'half' or 'interleaved'")
        if self.head_dim % 2:
            raise ValueError(f"rotary encoding needs an even head size, got {self.head_dim}")
        self.interleaved = pairing == "interleaved"
        j = torch.arange(0, self.head_dim // 2)
        theta = 1.0 / torch.pow(torch.tensor(float(p["base"])), (2 * j.float()) / self.head_dim)
        angle = torch.outer(torch.arange(self.max_context).float(), theta)
        self.table = torch.stack((torch.cos(angle), torch.sin(angle)), dim=-1).contiguous().to(ops.device)

    def rotary(self):
        return self.table, self.interleaved



@POSITION_ENCODINGS.register("none")
class NoPosition:
    """No position encoding: queries and keys go into attention as projected."""

    @classmethod
    def tensor_shapes(cls, params):
        return {}

    def __init__(self, spec, tensors, ops):
        self.max_context = int(spec.params.get("max_context", 1 << 30))

    def rotary(self):
        return None, False


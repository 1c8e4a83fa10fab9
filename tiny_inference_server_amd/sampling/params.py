"""Per-request sampling options, named as the reference's Request names them (server.py:79-87)."""
from __future__ import annotations

from dataclasses import dataclass


@dataclass(frozen=True)
class SamplingParams:
    max_new_tokens: int = 200
    temperature: float = 1.0     # 0 means greedy; the reference spells greedy as top_k=1 (test_server.py:110)
    top_k: int = 0               # 0: off
    top_p: float = 0.0           # 0: off
    rep_penalty: float = 1.0     # 1: off
    seed: int = 0                # the request's own random stream
    ignore_eos: bool = False

    def __post_init__(self):
        if self.max_new_tokens < 1:
            raise ValueError(f"max_new_tokens must be at least 1, got {self.max_new_tokens}")
        if self.temperature < 0:
            raise ValueError(f"temperature must not be negative, got {self.temperature}")
        if self.top_k < 0:
            raise ValueError(f"top_k must not be negative, got {self.top_k}")
        if not (0.0 <= self.top_p <= 1.0):
            raise ValueError(f"top_p must lie in [0, 1], got {self.top_p}")
        if self.rep_penalty <= 0:
            raise ValueError(f"rep_penalty must be positive, got {self.rep_penalty}")

    @property
    def greedy(self) -> bool:
        return self.temperature == 0.0 or self.top_k == 1

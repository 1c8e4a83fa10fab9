"""Sampling of one token per row of logits with the HIP sampling kernel.

Every request has a random stream of its own: the uniform number for its i-th generated token is a hash of
(seed, i), so a request's tokens do not depend on which other requests share its batch, nor on being
preempted and replayed. (The reference draws with torch.multinomial from the global generator,
server.py:240, which ties a request's tokens to the batch it happens to be in.)
"""
from __future__ import annotations

from typing import List, Sequence

import torch

from .params import SamplingParams

_MASK = (1 << 64) - 1


def uniform_for(seed: int, index: int) -> float:
    """A number in [0, 1) from (seed, index): the splitmix64 finaliser over a combined counter, top 24 bits."""
    z = (seed * 0x9E3779B97F4A7C15 + (index + 1) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    z ^= z >> 31
    return (z >> 40) / float(1 << 24)


class Sampler:
    def __init__(self, ops):
        self.ops = ops

    def sample(self, logits: torch.Tensor, params: Sequence[SamplingParams], token_index: Sequence[int],
               contexts: Sequence[Sequence[int]]) -> List[int]:
        """logits [n, vocab] float32 on the device; token_index[i]: how many tokens request i has generated so far;
        contexts[i]: its tokens so far, for the repetition penalty (server.py:29-36)."""
        n = logits.shape[0]
        if n == 0:
            return []
        dev = logits.device
        if all(p.greedy and p.rep_penalty == 1.0 for p in params):
            return self.ops.argmax(logits).tolist()
        f32 = lambda v: torch.tensor(v, dtype=torch.float32).to(dev)
        i32 = lambda v: torch.tensor(v, dtype=torch.int32).to(dev)
        uniform = [uniform_for(p.seed, i) for p, i in zip(params, token_index)]
        ctx_tokens = ctx_offsets = None
        if any(p.rep_penalty != 1.0 for p in params):
            flat, offs = [], [0]
            for p, c in zip(params, contexts):
                if p.rep_penalty != 1.0:
                    flat.extend(sorted(set(int(t) for t in c)))
                offs.append(len(flat))
            ctx_tokens, ctx_offsets = i32(flat if flat else [0]), i32(offs)
        out = self.ops.sample(logits, f32([p.temperature for p in params]), i32([p.top_k for p in params]),
                              f32([p.top_p for p in params]), f32([p.rep_penalty for p in params]), f32(uniform),
                              ctx_tokens, ctx_offsets)
        return out.tolist()

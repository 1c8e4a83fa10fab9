"""Sampling of one token per row of logits with the HIP sampling kernel.

Every request has a random stream of its own: the uniform number for its i-th generated token is a hash of
(seed, i), so a request's tokens do not depend on which other requests share its batch, nor on being
preempted and replayed. (The reference draws with torch.multinomial from the global generator,
server.py:240, which ties a request's tokens to the batch it happens to be in.)

For the repetition penalty the sampler keeps, per request slot, a table with one byte per token of the
vocabulary: a request's tokens are uploaded once, when it (re)enters, and the kernel itself marks every token
it draws. (The reference rebuilds a mask from every request's whole context at every step, server.py:29-36.)
"""
from __future__ import annotations

from typing import Hashable, List, Optional, Sequence

import numpy as np
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
    def __init__(self, ops, vocab_size: Optional[int] = None, max_requests: int = 0):
        self.ops = ops
        self.vocab_size = vocab_size
        self.max_requests = max_requests
        self.seen = None                 # [max_requests, vocab] bytes, made when a penalty is first asked for
        self._owner = {}                 # slot -> the (request, admission) whose tokens the slot's line holds

    def _line_for(self, slot: int, owner: Hashable, context: Sequence[int]) -> int:
        """The table line of `slot`, (re)filled from `context` if another request, or another admission, owned it."""
        if self.seen is None:
            self.seen = torch.zeros(self.max_requests, self.vocab_size, dtype=torch.uint8, device=self.ops.device)
        if self._owner.get(slot) != owner:
            self._owner[slot] = owner
            self.seen[slot].zero_()
            ids = torch.tensor(sorted(set(int(t) for t in context)), dtype=torch.long).to(self.ops.device)
            self.seen[slot, ids] = 1
        return slot

    def sample(self, logits: torch.Tensor, params: Sequence[SamplingParams], token_index: Sequence[int],
               contexts: Sequence[Sequence[int]], slots: Optional[Sequence[int]] = None,
               owners: Optional[Sequence[Hashable]] = None) -> List[int]:
        """logits [n, vocab] float32 on the device; token_index[i]: how many tokens request i has generated so far;
        contexts[i]: its tokens so far, for the repetition penalty (server.py:29-36). With `slots` (each row's
        request slot) and `owners` (something that changes when a slot changes hands) the contexts are kept on
        the device between steps; without, they are uploaded with the call."""
        n = logits.shape[0]
        if n == 0:
            return []
        dev = logits.device
        if all(p.greedy and p.rep_penalty == 1.0 for p in params):
            return self.ops.argmax(logits).tolist()
        penal = [p.rep_penalty != 1.0 for p in params]
        use_table = any(penal) and slots is not None and owners is not None and self.max_requests > 0 \
            and self.vocab_size == logits.shape[1]
        # every per-row parameter in one array, one copy: four rows of floats, two of integers
        packed = np.zeros((6, n), dtype=np.float32)
        packed[0] = [p.temperature for p in params]
        packed[1] = [p.top_p for p in params]
        packed[2] = [p.rep_penalty for p in params]
        packed[3] = [uniform_for(p.seed, i) for p, i in zip(params, token_index)]
        ints = packed.view(np.int32)
        ints[4] = [p.top_k for p in params]
        ints[5] = -1
        ctx_tokens = ctx_offsets = None
        if use_table:
            ints[5] = [self._line_for(s, o, c) if pen else -1 for s, o, c, pen in zip(slots, owners, contexts, penal)]
        elif any(penal):
            flat, offs = [], [0]
            for pen, c in zip(penal, contexts):
                if pen:
                    flat.extend(sorted(set(int(t) for t in c)))
                offs.append(len(flat))
            ctx_tokens = torch.tensor(flat if flat else [0], dtype=torch.int32).to(dev)
            ctx_offsets = torch.tensor(offs, dtype=torch.int32).to(dev)
        d = torch.from_numpy(packed).to(dev, non_blocking=True)
        di = d.view(torch.int32)
        out = self.ops.sample(logits, d[0], di[4], d[1], d[2], d[3], ctx_tokens, ctx_offsets,
                              self.seen if use_table else None, di[5] if use_table else None)
        return out.tolist()

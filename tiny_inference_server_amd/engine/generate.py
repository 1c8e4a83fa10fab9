"""The Python entry point: token ids in, generated token ids out."""
from __future__ import annotations

from typing import Optional, Sequence

from ..sampling.params import SamplingParams
from .engine import Engine
from .scheduler import Request, Scheduler


def generate(model, prompts: Sequence[Sequence[int]], max_new_tokens: int = 200, temperature: float = 1.0,
             top_k: int = 0, top_p: float = 0.0, rep_penalty: float = 1.0, seed: int = 0, ignore_eos: bool = False,
             dtype: str = "bfloat16", device: str = "cuda:0", max_batch: int = 8, token_budget: int = 2048,
             plan: str = "final", tokens_per_block: int = 16, pool_tokens: Optional[int] = None,
             params: Optional[Sequence[SamplingParams]] = None, return_scheduler: bool = False,
             run_heads: bool = False, static=None):
    """Generate for every prompt and return the new tokens, in the prompts' order.

    model: a model folder (config.json, model.safetensors) or an Engine already built. Request `i` draws from
    the random stream seed + i. pool_tokens: tokens the cache holds (default: room for max_batch full requests).
    run_heads: also run the multi-token-prediction heads at every step; their drafts are not used here, so by
    default generation runs the trunk alone (the reference's spec=False, server.py:106-118).
    static: None (pages on demand), "ctx", "req" or a number of tokens: pages taken at admission (server.py:107-111).
    """
    if isinstance(model, Engine):
        engine = model
    else:
        longest = max(len(p) for p in prompts) + max_new_tokens
        if pool_tokens is None:
            pool_tokens = max_batch * (-(-longest // tokens_per_block) * tokens_per_block)
        engine = Engine(model, dtype=dtype, page_size=tokens_per_block, max_tokens=pool_tokens,
                        max_requests=max_batch, device=device, run_heads=run_heads)
    sched = Scheduler(engine, max_batch=max_batch, token_budget=token_budget, plan=plan, static=static)
    reqs = []
    for i, p in enumerate(prompts):
        sp = params[i] if params is not None else SamplingParams(
            max_new_tokens=max_new_tokens, temperature=temperature, top_k=top_k, top_p=top_p,
            rep_penalty=rep_penalty, seed=seed + i, ignore_eos=ignore_eos)
        r = Request(p, sp)
        reqs.append(r)
        sched.submit(r)
    sched.run()
    outs = [r.out_ids() for r in reqs]
    return (outs, sched) if return_scheduler else outs

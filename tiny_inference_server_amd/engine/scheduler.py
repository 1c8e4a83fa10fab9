"""Continuous batching above the step function: admit, cut prompts into portions, decode, finish, free.

Follows the reference's scheduler (server.py:101-292, 475-479) where it has a rule, and adds what it lacks: a
token budget per step, under which prompts are fed in portions beside the decode tokens of other requests,
all in one batch (the reference prefills whole prompts in a launch of their own, server.py:279-284).

Admission (server.py:138-168): a queued request joins while a batch slot is free and the page plan allows.
plan "final" admits while every running request still fits at its full length (prompt + max_new_tokens), so
nothing is ever preempted; plan "cur" admits on what requests hold now, against a running budget, and lets
them outgrow the pool.

When pages run out (server.py:187-193, 261-269): before a step runs, while the step's new pages exceed the
free ones, the newest running request is taken out, its pages and state slot are given back, and it goes to
the front of the queue; later it is fed again from its prompt plus what it had generated, and its random
stream goes on where it was. A lone request that does not fit is an error.

Finishing (server.py:242-252): the end-of-sequence token, max_new_tokens, or the model's context.
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Deque, List, Optional, Sequence

from ..sampling.params import SamplingParams
from ..sampling.sampler import Sampler


class Request:
    _next_id = 0

    def __init__(self, prompt_ids: Sequence[int], params: Optional[SamplingParams] = None, **kw):
        if len(prompt_ids) == 0:
            raise ValueError("a request needs at least one prompt token")
        self.id = Request._next_id
        Request._next_id += 1
        self.ids: List[int] = [int(t) for t in prompt_ids]      # committed tokens: prompt + generated
        self.prompt_len = len(self.ids)
        self.params = params or SamplingParams(**kw)
        self.fed = 0            # positions whose keys and values are in the cache
        self.reserved = 0       # positions whose pages a static mode took at admission
        self.done = False
        self.preempted = 0

    def out_ids(self) -> List[int]:
        return self.ids[self.prompt_len:]

    @property
    def n_out(self) -> int:
        return len(self.ids) - self.prompt_len


@dataclass
class StepPlan:
    """What one step will run: (request, first position, number of tokens, sample afterwards?)."""
    items: List[tuple] = field(default_factory=list)

    @property
    def n_tokens(self) -> int:
        return sum(n for _, _, n, _ in self.items)


def pages_for(n_tokens: int, page_size: int) -> int:
    return -(-n_tokens // page_size)


class Scheduler:
    def __init__(self, engine, max_batch: int = 8, token_budget: int = 2048, plan: str = "final",
                 max_context: Optional[int] = None, static=None):
        """static: how pages are taken (reference server.py:107-111). None: on demand, as the request grows.
        "ctx": at admission, for the whole context; "req": for prompt plus max_new_tokens; an int: for that many
        tokens. A request with a reservation never has to be preempted for pages it already holds."""
        if plan not in ("final", "cur"):
            raise ValueError(f"plan {plan!r}: use 'final' or 'cur'")
        if not (static is None or static in ("ctx", "req") or (isinstance(static, int) and static > 0)):
            raise ValueError(f"static {static!r}: use None, 'ctx', 'req' or a number of tokens")
        if max_batch < 1:
            raise ValueError(f"max_batch must be at least 1, got {max_batch}")
        if token_budget < max_batch:
            raise ValueError(f"token_budget {token_budget} must give every one of {max_batch} requests a token")
        self.engine = engine
        self.max_batch = min(max_batch, engine.cache.max_requests)
        self.token_budget = token_budget
        self.plan = plan
        self.static = static
        self.max_context = min(max_context or engine.spec.max_context, engine.spec.max_context)
        self.eos = engine.spec.eos_token_id
        self.page_size = engine.page_size
        self.sampler = Sampler(engine.ops, engine.spec.vocab_size, engine.cache.max_requests)
        self.queue: Deque[Request] = deque()
        self.active: List[Request] = []
        self.finished: List[Request] = []
        self.preempts = 0
        self.replays = 0            # preempted after work was done: that work is done again
        self.peak_running = 0
        self.steps = 0
        self.tokens_run = 0
        self.last_plan: Optional[StepPlan] = None       # what the latest step ran, for whoever measures steps

    # ---- queueing and admission ----------------------------------------------------------------------
    def submit(self, req: Request) -> None:
        if req.prompt_len >= self.max_context:
            raise ValueError(f"a prompt of {req.prompt_len} tokens leaves no room in a context of {self.max_context}")
        self.queue.append(req)

    # How many pages something takes is the engine's knowledge (its cache manager's groups: all keys, a window of
    # them, none at all); the scheduler only adds, compares and decides.
    def _grow_pages(self, r: Request, n_new: int) -> int:
        """Pages r must take to be fed n_new more tokens (a request is known to the engine from its first step, or
        from a static reservation, on)."""
        if r.id in self.engine.requests:
            return self.engine.pages_to_grow(r.id, n_new)
        return self.engine.pages_to_hold(r.fed + n_new, n_new)

    def _pages_for(self, n_tokens: int) -> int:
        """Pages a request of n_tokens holds at the most, fed under this scheduler's token budget."""
        return self.engine.pages_to_hold(n_tokens, self.token_budget)

    def _reserve_tokens(self, r: Request) -> int:
        """Tokens a static mode reserves at admission (reference server.py:180-185)."""
        if self.static == "ctx":
            return self.max_context
        if self.static == "req":
            return min(r.prompt_len + r.params.max_new_tokens, self.max_context)
        return min(int(self.static), self.max_context)

    def _final_pages(self, r: Request) -> int:
        """Pages r holds once it has generated all it may (the last token is sampled, never fed)."""
        return self._pages_for(min(r.prompt_len + r.params.max_new_tokens - 1, self.max_context))

    def admit(self) -> None:
        total = self.engine.total_pages()
        # pages are only taken when a request runs, so the free count does not move while admitting: keep a
        # budget instead (the reference's fix, server.py:143-147)
        budget = self.engine.free_pages() - sum(self._grow_pages(r, len(r.ids) - r.fed) for r in self.active)
        while self.queue and len(self.active) < self.max_batch:
            q = self.queue[0]
            tokens_now = max(len(q.ids), self._reserve_tokens(q)) if self.static else len(q.ids)
            # (a reservation takes every position's page, also where a window would give pages back)
            need_now = self.engine.pages_to_hold(tokens_now, tokens_now) if self.static else self._pages_for(tokens_now)
            if self.static and need_now > total:
                raise RuntimeError(f"static reservation {need_now} pages > pool {total}")
            if self.plan == "final" and not self.static:
                projected = sum(self._final_pages(r) for r in self.active) + self._final_pages(q)
                if projected > total and self.active:
                    break
            elif need_now > budget and (self.active or self.static):
                break
            budget -= need_now
            self.queue.popleft()
            q.fed = 0
            q.reserved = 0
            if self.static:
                # every page now, so that this request never needs another (reference server.py:163-166)
                q.reserved = need_now * self.page_size
                self.engine.reserve(q.id, q.reserved)
            self.active.append(q)

    # ---- one step ------------------------------------------------------------------------------------
    def plan_step(self) -> StepPlan:
        """Decode tokens first, then prompt portions in admission order, under the token budget."""
        plan = StepPlan()
        left = self.token_budget
        for r in self.active:
            if len(r.ids) - r.fed == 1 and r.fed >= r.prompt_len:
                plan.items.append((r, r.fed, 1, True))
                left -= 1
        for r in self.active:
            pending = len(r.ids) - r.fed
            if pending >= 1 and not (pending == 1 and r.fed >= r.prompt_len):
                if left <= 0:
                    continue
                n = min(pending, left)
                plan.items.append((r, r.fed, n, n == pending))
                left -= n
        return plan

    def preempt(self) -> None:
        r = self.active.pop()
        self.preempts += 1
        if r.fed > 0:
            self.replays += 1
        if r.id in self.engine.requests:
            self.engine.close(r.id)
        r.fed = 0
        r.reserved = 0
        r.preempted += 1
        self.queue.appendleft(r)

    def step(self) -> None:
        if not self.active:
            return
        while True:
            plan = self.plan_step()
            need = sum(self._grow_pages(r, n) for r, _, n, _ in plan.items)
            if need <= self.engine.free_pages():
                break
            if len(self.active) == 1:
                r = self.active[0]
                raise RuntimeError("kv pool too small for a single request: "
                                   f"{len(r.ids)} tokens need {self._pages_for(len(r.ids))} pages of "
                                   f"{self.page_size}, the pool has {self.engine.total_pages()}")
            self.preempt()
        self.peak_running = max(self.peak_running, len(self.active))
        self.last_plan = plan
        if not plan.items:
            return
        entries = []
        for r, start, n, sample in plan.items:
            entries.append((r.id, r.ids[start:start + n], [n - 1] if sample else []))
        out = self.engine.step(entries)
        self.steps += 1
        self.tokens_run += plan.n_tokens
        sampled = [r for r, _, _, s in plan.items if s]
        for r, _, n, _ in plan.items:
            r.fed += n
        if sampled:
            toks = self.sampler.sample(out.logits, [r.params for r in sampled],
                                       [r.n_out for r in sampled], [r.ids for r in sampled],
                                       slots=[self.engine.requests[r.id][0] for r in sampled],
                                       owners=[(r.id, r.preempted) for r in sampled])
            for r, t in zip(sampled, toks):
                r.ids.append(int(t))
                self.finish_check(r)
        for r in self.active:
            if r.done:
                self.engine.close(r.id)
                self.finished.append(r)
        self.active = [r for r in self.active if not r.done]

    def finish_check(self, r: Request) -> None:
        """Called after every token appended to r: only the last one can be new."""
        if self.eos >= 0 and not r.params.ignore_eos and r.n_out > 0 and r.ids[-1] == self.eos:
            r.done = True
        if r.n_out >= r.params.max_new_tokens:
            del r.ids[r.prompt_len + r.params.max_new_tokens:]
            r.done = True
        if len(r.ids) >= self.max_context:
            r.done = True

    def run(self) -> List[Request]:
        while self.queue or self.active:
            self.admit()
            if not self.active:
                raise RuntimeError("nothing can be admitted: is max_batch 0 or the pool empty?")
            self.step()
        return self.finished

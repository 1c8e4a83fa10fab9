"""A model built from a spec of parts, and the pass that runs a step's rows through it.

Nothing here knows an architecture: the spec says which layers exist, in which order each stage calls
them, whose cache a call uses, where a stage's rows come from and which norm closes it.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..parts.base import ARRANGEMENTS, CallContext, Tensors, build_part, part_class, to_compute
from ..parts.spec import ModelSpec, PagedKvNeed, StateNeed


class StageOutput:
    def __init__(self, hidden, batch):
        self.hidden = hidden        # [rows, d_model], after the stage's closing norm
        self.batch = batch


class Model:
    def __init__(self, spec: ModelSpec, tensors: Dict[str, torch.Tensor], ops):
        self.spec, self.ops = spec, ops
        T = Tensors(tensors)
        self.layers = [ARRANGEMENTS.get(ls.arrangement)(ls, T, ops) for ls in spec.layers]
        self.inputs = [build_part(st.input, T, ops) for st in spec.stages]
        self.out_norms = [build_part(st.out_norm, T, ops) for st in spec.stages]
        emb = to_compute(ops, tensors[spec.embedding])
        self.shared = {"embedding": emb,
                       "lm_head": emb if spec.lm_head == spec.embedding else to_compute(ops, tensors[spec.lm_head])}
        # a step may be captured as a graph only if every part promises that what it launches depends on the
        # step's device arrays alone, never on host values that change from step to step
        parts = list(self.inputs) + list(self.out_norms)
        for blk in self.layers:
            # an arrangement that builds no parts of its own answers for itself
            parts += list(getattr(blk, "parts", {}).values()) or [blk]
        # (a part may promise it for steps of single rows only, "single_rows": a recurrence that walks a portion's rows
        # on the host, but updates its state with device arrays alone when every request brings one token)
        self.graph_safe = all(getattr(p, "graph_safe", False) is True for p in parts)
        self.graph_safe_single_rows = all(getattr(p, "graph_safe", False) in (True, "single_rows") for p in parts)
        # host planning that parts ask for, once per distinct key (layers of one shape share a plan)
        self._planners = {}
        for p in parts:
            key = p.plan_key() if hasattr(p, "plan_key") else None
            if key is not None:
                self._planners.setdefault(key, p)
        self.lags = [st.lag for st in spec.stages]
        self.max_lag = max(self.lags)
        self.reads_previous = [bool(getattr(part_class(st.input), "reads_previous", False)) for st in spec.stages]
        if self.reads_previous and self.reads_previous[0]:
            raise ValueError("the first stage cannot read a previous stage")
        # cache keys: one per call and mixer part unless the call names another's; a block with one mixer uses the
        # call's key as it is, a block with several appends the part's name
        self.call_keys: List[List[Dict[str, str]]] = []
        self.needs: Dict[str, object] = {}
        for st in spec.stages:
            keys = []
            for i, call in enumerate(st.calls):
                base = call.cache or f"{st.name}.{i}"
                mixers = spec.layers[call.layer].mixers()
                per_part = {}
                for name, mixer in mixers:
                    key = base if len(mixers) == 1 else f"{base}:{name}"
                    need = part_class(mixer).cache_need(mixer.params)
                    if call.writes_cache or key not in self.needs:
                        if key in self.needs and self.needs[key] != need:
                            raise ValueError(f"cache {key!r} is shared by layers that need different things: "
                                             f"{self.needs[key]} and {need}")
                        if need is not None:
                            self.needs[key] = need
                    per_part[name] = key
                keys.append(per_part)
            self.call_keys.append(keys)
        self.state_keys: List[Optional[str]] = []
        for st in spec.stages:
            need = part_class(st.input).state_need(st.input.params)
            key = (st.state_key or f"{st.name}.input") if need is not None else None
            if key is not None:
                self.needs[key] = need
            self.state_keys.append(key)

    def cache_needs(self) -> Dict[str, object]:
        return dict(self.needs)

    def plan_mode(self, seq_rows):
        """What kind of plans a step gets, decided once from the first stage's rows (first row, first position, rows
        per request) and handed to plan_rows for every stage: hashable, and part of what must be equal for two steps
        to share a captured graph. None: nothing to say."""
        modes = tuple((key, part.plan_mode(seq_rows)) for key, part in self._planners.items() if hasattr(part, "plan_mode"))
        modes = tuple(m for m in modes if m[1] is not None)
        return modes or None

    def plan_rows(self, seq_rows, add, mode=None):
        """Host planning of every part that asks for it, for one stage's rows: {name: (packed array id, values...)}."""
        plans = {}
        of = dict(mode) if mode else {}
        for key, part in self._planners.items():
            plans.update(part.plan_rows(seq_rows, add, of[key]) if key in of else part.plan_rows(seq_rows, add))
        return plans

    def _bind(self, ctx, key, cache):
        need = self.needs.get(key)
        if isinstance(need, PagedKvNeed):
            ctx.group = cache.group_of[key]
            ctx.plane = cache.groups[ctx.group].plane(key)
        elif isinstance(need, StateNeed):
            ctx.state = cache.states[key]
        return ctx

    def _run_stage(self, j, step, cache, prev):
        st, b = self.spec.stages[j], step.stages[j]
        state = cache.states.get(self.state_keys[j]) if self.state_keys[j] else None
        x = self.inputs[j].forward(b, prev, self.shared, state)
        if b.n_rows:
            for i, call in enumerate(st.calls):
                keys = self.call_keys[j][i]
                # the rows going into a layer are replaced by its result: the layer may overwrite them
                ctx = CallContext(batch=b, writes_cache=call.writes_cache, residual_is_spent=True)
                if len(keys) == 1:
                    self._bind(ctx, next(iter(keys.values())), cache)
                elif keys:
                    ctx.bindings = {name: self._bind(CallContext(batch=b, writes_cache=call.writes_cache), key, cache)
                                    for name, key in keys.items()}
                x = self.layers[call.layer].forward(x, ctx)
            x = self.out_norms[j](x)
        return x

    def forward(self, step, cache) -> List[StageOutput]:
        """Run every stage over its rows; keys, values and state land in `cache`.

        A stage that reads the previous one takes each row either from that stage's rows of this step or from
        the request's state (a row made one step earlier); what a stage keeps for the next step is written after
        all stages have read. The stages run one after the other on one stream, also in steps of single decoded
        tokens where they do not depend on one another: as branches of a captured graph they measured slower
        on MI355X than in sequence (4.3k against 4.5k tokens a second at batch 8).
        """
        n = len(self.spec.stages)
        hidden = [None] * n
        for j in range(n):
            hidden[j] = self._run_stage(j, step, cache, hidden[j - 1] if j else None)
        for j in range(1, n):
            after = getattr(self.inputs[j], "after_step", None)
            if after is not None:
                after(step.stages[j], hidden[j - 1], cache.states.get(self.state_keys[j]) if self.state_keys[j] else None)
        return [StageOutput(hidden[j], step.stages[j]) for j in range(n)]

    def _wanted_rows(self, hidden, want_index, n, out=None):
        return self.ops.gather_rows(hidden, hidden, want_index[:n], out=out)

    def _project(self, rows):
        """Rows after a stage's closing norm -> 32-bit logits: the one place the output table is applied."""
        return self.ops.linear(rows, self.shared["lm_head"], out_dtype=torch.float32)

    def logits(self, hidden, want_index, n):
        """32-bit logits [n, vocab] of the rows `want_index` of `hidden` (reference main_models_new.py:225-226)."""
        return self._project(self._wanted_rows(hidden, want_index, n))

    def logits_of_stages(self, outs, n):
        """Logits of every stage at the n wanted places from one product with the output table, which all stages
        share (reference main_models_new.py:225-226): the table is read once however many stages there are.
        Returns (first stage's logits [n, vocab], [logits of each further stage], [which of their rows are valid]);
        rows that a later stage does not have yet come back as NaN. The first stage's part is what `logits` gives: the
        same gather and the same product on the same rows (up to the order of 32-bit partial sums, which the product
        may choose by the number of rows)."""
        vocab, S = self.spec.vocab_size, len(outs)
        if n == 0:
            e = torch.empty(0, vocab, dtype=torch.float32, device=self.ops.device)
            return e, [e.clone() for _ in outs[1:]], [[] for _ in outs[1:]]
        rows = self.ops.empty(S * n, self.spec.d_model)
        valid = []
        for j, o in enumerate(outs):
            v = [True] * n if j == 0 else list(o.batch.want_valid)
            part = rows[j * n:(j + 1) * n]
            if o.batch.n_rows and any(v):
                idx = o.batch.want_index[:n] if j == 0 else torch.clamp(o.batch.want_index[:n], min=0)
                self._wanted_rows(o.hidden, idx, n, out=part)
            else:
                part.zero_()
            valid.append(v)
        lg = self._project(rows).view(S, n, vocab)
        later = []
        for j in range(1, S):
            h = lg[j]
            if not all(valid[j]):
                h[~torch.tensor(valid[j], device=self.ops.device)] = float("nan")
            later.append(h)
        return lg[0], later, valid[1:]

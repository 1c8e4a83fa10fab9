#!/usr/bin/env python3
"""Decode and prefill throughput of the engine on one MI355X, with random weights.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--size 0.9B] [--batch 8] [--context 4096]

A step is one decode step: every live request advances by one token through the whole model (trunk, the
prediction heads unless --trunk-only, output table, sampling, read-back of the tokens). One JSON line is
printed: decoded tokens a second at the given batch, the prefill of 2,048 tokens, the decode step's
bandwidth against the HBM peak, and under `points`: decode at batch 1, 16, 32 and 64 (each with its fraction of the
HBM peak), decode at context 8,192 (the longest the size's position table allows), a prefill of 8,192 tokens, the
same batch-8 decode without the prediction heads and driven by the scheduler with the reference's sampling options
instead of by the step function with arg-max, and the serve workload below.

Two more workloads run whole requests through the scheduler (admission, portions under the token budget, sampling
with temperature, top-k, top-p and repetition penalty, finishing, pages given back):

    python bench.py --workload serve --size 2.1B     64 requests at once, prompts of 128..4096 tokens, 256 new each
    python bench.py --workload mixed --size 2.1B     64 requests decoding at contexts of 512..8192 while 2,048-token
                                                     portions of further prompts run in the same steps

Each prints one line of the same form; `value` is generated tokens a second over the whole run (serve) or over the
steps that hold 64 decoding requests and a portion (mixed), `roofline` the sum of the steps' floors (the larger of
bytes / HBM peak and flops / matrix peak) over the sum of their times.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# MI355X published peaks
HBM_GBS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}
# the reference's plain decode at batch 8 on an A6000: 31.7 ms per iteration of 8 tokens (README.md:325)
REFERENCE_B8_TOKS = 8 / 31.7e-3


class Costs:
    """What a step of a model costs, read from the engine's own description of the model (the spec's tensors, the
    stages' run order, the cache manager's groups): nothing here names an architecture's configuration fields."""

    def __init__(self, engine):
        from tiny_inference_server_amd.weights.loader import spec_tensors
        spec = engine.run_spec
        shapes = spec_tensors(spec)
        called = {call.layer for st in spec.stages for call in st.calls}
        names = set()
        for i, layer in enumerate(spec.layers):
            if i in called:
                for part in layer.parts.values():
                    names.update(_tensor_names(part))
        for st in spec.stages:
            names.update(_tensor_names(st.input))
        count = lambda ns: sum(shapes[n][0] * shapes[n][1] for n in ns if len(shapes[n]) == 2)
        # matrices a step reads once: every called layer's and stage input's, and the output table (the token table
        # is only gathered from, unless it is the output table too)
        self.matrix_elems = count(names - {spec.embedding, spec.lm_head})
        self.table_elems = shapes[spec.lm_head][0] * shapes[spec.lm_head][1]
        self.kv_bytes_per_token = engine.cache.bytes_per_position()
        # attention: 4 flops per (row, key) pair, query head and head element, for every call of a mixer that has them
        self.attn_flops_per_pair = 0.0
        for st in spec.stages:
            for call in st.calls:
                for _, mixer in spec.layers[call.layer].mixers():
                    if "n_heads" in mixer.params and "head_dim" in mixer.params:
                        self.attn_flops_per_pair += 4.0 * mixer.params["n_heads"] * mixer.params["head_dim"]
        self.elem = 2 if engine.dtype.itemsize == 2 else 4

    def step_bytes(self, kv_tokens: float) -> float:
        return (self.matrix_elems + self.table_elems) * self.elem + kv_tokens * self.kv_bytes_per_token

    def step_flops(self, n_tokens: float, attn_pairs: float, table_rows: float = 0.0) -> float:
        return 2.0 * self.matrix_elems * n_tokens + 2.0 * self.table_elems * table_rows + self.attn_flops_per_pair * attn_pairs

    def prefill_flops(self, T: int) -> float:
        return self.step_flops(T, T * (T + 1) / 2, table_rows=1)      # the output table runs for one row

    def step_floor(self, n_tokens, kv_tokens, attn_pairs, dkey):
        """Seconds one step needs at the least: its bytes at the HBM peak or its flops at the matrix peak."""
        byts, flops = self.step_bytes(kv_tokens), self.step_flops(n_tokens, attn_pairs)
        return max(byts / (HBM_GBS * 1e9), flops / PEAK_FLOPS[dkey]), byts, flops


def _tensor_names(part):
    names = set(part.tensors.values())
    for v in part.params.values():
        if hasattr(v, "tensors") and hasattr(v, "params"):
            names |= _tensor_names(v)
    return names


def model_sizes(engine):
    """The sizes a result line names, flat: from the spec and its parts' parameters, whatever the architecture."""
    spec = engine.run_spec
    out = {"n_layers": len({c.layer for c in spec.stages[0].calls}), "d_model": spec.d_model, "vocab_size": spec.vocab_size}
    mixers = [m for c in spec.stages[0].calls for _, m in spec.layers[c.layer].mixers()]
    for key in ("n_heads", "n_kv_heads", "head_dim"):
        vals = {m.params[key] for m in mixers if key in m.params}
        if len(vals) == 1:
            out[key] = vals.pop()
    ffn = {p.params["hidden"] for c in spec.stages[0].calls for p in spec.layers[c.layer].parts.values()
           if p.role == "feed_forward" and "hidden" in p.params}
    if len(ffn) == 1:
        out["ffn_hidden"] = ffn.pop()
    out["tie_embeddings"] = spec.embedding == spec.lm_head
    out["mtp_heads_run"] = len(spec.stages) - 1
    return out


# the reference's sampling options for its runs (server.py:515-516, evals.py:120)
SAMPLING = dict(temperature=0.9, top_k=50, top_p=0.95, rep_penalty=1.1)


def scheduler_decode_rate(engine, a, gen):
    """Tokens a second of `a.steps` decode steps at batch `a.batch` near the context length, through the scheduler."""
    import torch

    from tiny_inference_server_amd.engine.scheduler import Request, Scheduler
    from tiny_inference_server_amd.sampling.params import SamplingParams
    sched = Scheduler(engine, max_batch=a.batch, token_budget=2048 + a.batch, plan="final")
    # a request that has its prompt in decodes while the others' portions are still fed: room for those tokens too
    early = a.batch * -(-a.context // 2048) + 2
    start_len = max(1, a.context - a.steps - a.warmup - early)
    for i in range(a.batch):
        ids = torch.randint(0, engine.spec.vocab_size, (start_len,), generator=gen).tolist()
        sched.submit(Request(ids, SamplingParams(max_new_tokens=a.steps + a.warmup + early, seed=a.seed + i,
                                                 ignore_eos=True, **SAMPLING)))
    sched.admit()
    while any(r.fed < r.prompt_len for r in sched.active):      # prompts, in portions; the last portion samples
        sched.step()
    for _ in range(a.warmup):
        sched.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(a.steps):
        sched.step()
        assert len(sched.last_plan.items) == a.batch and sched.last_plan.n_tokens == a.batch
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    sched.run()
    return a.batch * a.steps / dt


def scheduler_workload(a, cfg, layers_full, tensors, heads, page, say, workload=None):
    """Whole requests through the scheduler: `serve` and `mixed` (see the top of the file). Returns the result line."""
    workload = workload or a.workload
    import random

    import torch

    from tiny_inference_server_amd.engine import Engine
    from tiny_inference_server_amd.engine.scheduler import Request, Scheduler
    from tiny_inference_server_amd.sampling.params import SamplingParams
    dev = "cuda:0"
    rng = random.Random(a.seed)
    gen = torch.Generator().manual_seed(a.seed)
    dkey = "bf16" if a.dtype == "bfloat16" else "fp32"
    n_req, portion = a.requests, a.prefill_tokens
    from tiny_inference_server_amd.config import ARCHITECTURES
    spec = ARCHITECTURES.get(cfg.architecture).build_spec(cfg)
    context, vocab = min(spec.max_context, 8192), spec.vocab_size

    def ids_of(n):
        return torch.randint(0, vocab, (n,), generator=gen).tolist()

    if workload == "serve":
        new = a.new_tokens
        longest = min(4096, context - new - 1)
        lens = [rng.randint(min(128, longest), longest) for _ in range(n_req)]
        pool = sum(-(-(n + new) // page) * page for n in lens)
        extra_slots = 0
    else:
        # a request whose prompt is in decodes while the others' prompts are still fed: room for those tokens too
        new = a.steps + a.warmup + 8 + n_req * (context // portion + 1)
        if new + 2 > context:
            raise ValueError(f"a context of {context} has no room for {new} decoded tokens")
        lens = [rng.randint(min(512, context - new - 1), context - new - 1) for _ in range(n_req)]
        pool = sum(-(-(n + new) // page) * page for n in lens) + 2 * context
        extra_slots = 1
    engine = Engine(config=cfg, tensors=tensors, dtype=a.dtype, page_size=page, max_tokens=pool,
                    max_requests=n_req + extra_slots, device=dev, run_heads=heads)
    sched = Scheduler(engine, max_batch=n_req + extra_slots, token_budget=portion + n_req, plan="final",
                      max_context=context)
    records = []        # (seconds, tokens, decoding requests, tokens held by the step's requests, attention pairs)

    def timed_step():
        torch.cuda.synchronize()
        replays = engine.graph_replays
        t0 = time.perf_counter()
        sched.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        items = sched.last_plan.items
        kv = sum(start + n for _, start, n, _ in items)
        pairs = sum(n * start + n * (n + 1) / 2 for _, start, n, _ in items)
        n_dec = sum(1 for r, start, n, _ in items if n == 1 and start >= r.prompt_len)
        records.append((dt, sum(n for _, _, n, _ in items), n_dec, kv, pairs, engine.graph_replays > replays))

    def params(i, n_new):
        return SamplingParams(max_new_tokens=n_new, seed=a.seed + i, ignore_eos=True, **SAMPLING)

    if workload == "serve":
        say(f"serve: {n_req} requests, prompts of {min(lens)}..{max(lens)} tokens ({sum(lens)} in all), {new} new each")
        # a short run of the same kind first: the library's set-up and the first captures are not the workload's
        for i in range(4):
            sched.submit(Request(ids_of(min(300 + 40 * i, context // 2)), params(i, 8)))
        sched.run()
        sched.finished.clear()
        for i, n in enumerate(lens):
            sched.submit(Request(ids_of(n), params(i, new)))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        while sched.queue or sched.active:
            sched.admit()
            timed_step()
        wall = time.perf_counter() - t0
        generated = sum(len(r.out_ids()) for r in sched.finished)
        assert generated == n_req * new, (generated, n_req * new)
        value, timed = generated / wall, records
        dec = [r for r in records if r[2] == r[1]]                 # steps of decoded tokens only
        eager = [r for r in dec if not r[5]]                       # a shape's first steps: run as they are, or captured
        detail = {"wall_s": round(wall, 3), "steps": len(records), "decode_only_steps": len(dec),
                  "decode_only_ms": round(1e3 * sum(r[0] for r in dec) / max(1, len(dec)), 3),
                  "decode_only_steps_not_replayed": len(eager),
                  "decode_only_ms_not_replayed": round(1e3 * sum(r[0] for r in eager) / max(1, len(eager)), 3),
                  "prompt_tokens": sum(lens), "generated_tokens": generated, "preemptions": sched.preempts,
                  "all_tokens_per_s": round((sum(lens) + generated) / wall, 1)}
    else:
        say(f"mixed: {n_req} requests decoding at contexts of {min(lens)}..{max(lens)} tokens, "
            f"{portion}-token portions of further prompts beside them")
        for i, n in enumerate(lens):
            sched.submit(Request(ids_of(n), params(i, new)))
        sched.admit()
        while any(r.fed < r.prompt_len for r in sched.active):
            sched.step()
        records.clear()
        # from here on a further prompt is always being fed: each takes the free slot, runs its portions beside the
        # decoded tokens, generates one token and leaves
        long_prompt = (context - 2) // portion * portion
        n_steps = a.steps + a.warmup
        k = 0
        while len(records) < n_steps:
            if not sched.queue and len(sched.active) <= n_req:
                sched.submit(Request(ids_of(long_prompt), params(n_req + k, 1)))
                k += 1
            sched.admit()
            timed_step()
        timed = [r for r in records[a.warmup:] if r[2] == n_req and r[1] == n_req + portion]
        if not timed:
            raise RuntimeError("no step held the decoding requests and a whole portion")
        seconds = sum(r[0] for r in timed)
        value = n_req * len(timed) / seconds
        detail = {"timed_steps": len(timed), "ms_per_mixed_step": round(1e3 * seconds / len(timed), 3),
                  "portion_tokens_per_s": round(portion * len(timed) / seconds, 1),
                  "mean_context": round(sum(lens) / n_req, 1)}
    costs = Costs(engine)
    floors = [costs.step_floor(r[1], r[3], r[4], dkey) for r in timed]
    floor_s, meas_s = sum(f[0] for f in floors), sum(r[0] for r in timed)
    byts, flops = sum(f[1] for f in floors), sum(f[2] for f in floors)
    line = {
        "metric": f"generated tok/s, workload {workload} ({a.size}, {dkey}, {n_req} requests through the scheduler)",
        "value": round(value, 1), "unit": "tok/s", "n_gpus": 1, "steps": len(timed), "warmup": a.warmup,
        "ms_per_step": round(1e3 * meas_s / len(timed), 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": dkey, "data": "synthetic: random weights N(0,0.02), uniform random token ids",
        "config": {
            "model": a.size, "workload": workload, "global_batch": n_req, "seq_len": context,
            "parallelism": "single-gpu", **model_sizes(engine), "n_layers_full": layers_full,
            "mtp_head_logits": False, "page_size": page, "token_budget": portion + n_req,
            "sampling": "temperature 0.9, top-k 50, top-p 0.95, repetition penalty 1.1",
        },
        "roofline": {"bound": "hbm or mfma per step", "achieved": round(floor_s / meas_s, 4), "peak": 1.0,
                     "unit": "sum of step floors / sum of step times", "frac": round(floor_s / meas_s, 4),
                     "hbm_GBs": round(byts / meas_s / 1e9, 1), "mfma_TFLOPs": round(flops / meas_s / 1e12, 1)},
        "detail": detail,
    }
    return line


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--size", default="0.9B")
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the size has (0: all)")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    ap.add_argument("--trunk-only", action="store_true", help="leave the prediction heads out, as the reference's plain decode does")
    ap.add_argument("--points", default="1,16,32,64", help="other batch sizes to measure, comma separated ('' for none)")
    ap.add_argument("--context-points", default="8192", help="other context lengths for decode at the given batch and at 64 ('' for none)")
    ap.add_argument("--prefill-points", default="8192", help="other prompt lengths for the prefill ('' for none)")
    ap.add_argument("--no-serve-point", dest="serve_point", action="store_false",
                    help="skip the serve workload's figure in `points`")
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--no-trunk-point", dest="trunk_point", action="store_false",
                    help="skip the extra decode measurement without the prediction heads")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--workload", choices=["decode", "serve", "mixed"], default="decode")
    ap.add_argument("--requests", type=int, default=64, help="serve, mixed: requests (decoding at once)")
    ap.add_argument("--new-tokens", type=int, default=256, help="serve: tokens generated per request")
    a = ap.parse_args()
    if a.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {a.gpus} is not supported")
        return 2
    if a.size == "7B":
        print("bench.py: --size 7B is switched off for every workload: its widths are not among those the library's "
              "matrix product is used at (tiny_inference_server_amd/ops/library_widths.json), and runs at that size "
              "have ended with the GPU faulted", file=sys.stderr)
        return 2

    import dataclasses

    import torch

    from tiny_inference_server_amd.__main__ import size_config
    from tiny_inference_server_amd.engine import Engine
    from tiny_inference_server_amd.weights import random_tensors

    def say(what):
        # progress on stderr, flushed: names the phase a run was in if it ends without its line
        print(f"[bench] {what}", file=sys.stderr, flush=True)

    # the library's product kernels differ from shape to shape: each new shape is named on stderr before its first launch
    os.environ.setdefault("TIS_TRACE_SHAPES", "1")

    from tiny_inference_server_amd.config import ARCHITECTURES

    cfg_full = size_config(a.size)
    cfg = cfg_full
    spec_full = ARCHITECTURES.get(cfg_full.architecture).build_spec(cfg_full)
    layers_full = len(spec_full.stages[0].calls)
    if a.layers and a.layers != layers_full:
        # (fewer layers is a matter of the architecture's own configuration: asked of one that has such a field)
        cfg = dataclasses.replace(cfg_full, n_layers=a.layers)
    heads = len(spec_full.stages) > 1 and not a.trunk_only
    dev = "cuda:0"
    torch.cuda.set_device(0)
    tensors = random_tensors(cfg, a.seed, dtype=a.dtype, device=dev)
    page = 16
    if a.workload != "decode":
        print(json.dumps(scheduler_workload(a, cfg, layers_full, tensors, heads, page, say)))
        return 0
    points = [int(p) for p in a.points.split(",") if p.strip()]
    contexts = [int(c) for c in a.context_points.split(",") if c.strip()]
    too_long = [c for c in contexts if c > spec_full.max_context]
    if too_long:
        # the position table ends at the model's context: no point beyond it
        say(f"contexts {too_long} are beyond the model's {spec_full.max_context}: left out")
        contexts = [c for c in contexts if c <= spec_full.max_context]
    max_b = max([a.batch] + points)
    pool = max([max_b * (a.context + page)] + [max(a.batch, 64 if 64 in points else a.batch) * (c + page) for c in contexts])
    engine = Engine(config=cfg, tensors=tensors, dtype=a.dtype, page_size=page, max_tokens=pool, max_requests=max_b,
                    device=dev, run_heads=heads)
    trunk = None
    if heads and a.trunk_point:
        trunk = Engine(config=cfg, tensors=tensors, dtype=a.dtype, page_size=page,
                       max_tokens=a.batch * (a.context + page), max_requests=a.batch, device=dev, run_heads=False)
    vocab = engine.spec.vocab_size
    gen = torch.Generator().manual_seed(a.seed)
    costs = Costs(engine)

    def decode_rate(B: int, steps: int, warmup: int, engine=engine, context=a.context):
        """Tokens a second and seconds per step of `steps` decode steps at batch B near the context length."""
        start_len = context - steps - warmup - 1
        rids = [f"b{B}_{context}_{i}" for i in range(B)]
        for rid in rids:
            ids = torch.randint(0, vocab, (start_len,), generator=gen).tolist()
            for p in range(0, start_len, 2048):
                engine.step([(rid, ids[p:p + 2048], [])])
        toks = torch.randint(0, vocab, (B,), generator=gen).tolist()

        def one(toks):
            out = engine.step([(rid, [t], [0]) for rid, t in zip(rids, toks)])
            return engine.ops.argmax(out.logits).tolist()
        for _ in range(warmup):
            toks = one(toks)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            toks = one(toks)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        for rid in rids:
            engine.close(rid)
        return B * steps / dt, dt / steps

    def prefill_rate(T: int, reps: int = 5):
        ids = torch.randint(0, vocab, (T,), generator=gen).tolist()
        best = None
        for i in range(reps + 1):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            out = engine.step([("prefill", ids, [T - 1])])
            engine.ops.argmax(out.logits).tolist()
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            engine.close("prefill")
            if i > 0:                               # the first run warms up
                best = dt if best is None else min(best, dt)
        return best

    def hbm_frac(B, context, steps, sec_per_step):
        """The decode step's bytes (every weight once, the live requests' keys and values) / its time / the HBM peak."""
        return costs.step_bytes(B * (context - steps // 2)) / sec_per_step / 1e9 / HBM_GBS

    sizes = model_sizes(engine)
    say(f"{a.size}, {sizes['n_layers']} layers, {a.dtype}: decode at batch {a.batch}, context {a.context}")
    value, sec_per_step = decode_rate(a.batch, a.steps, a.warmup)
    achieved = costs.step_bytes(a.batch * (a.context - a.steps // 2)) / sec_per_step / 1e9
    say(f"prefill of {a.prefill_tokens} tokens")
    pt = prefill_rate(a.prefill_tokens)
    dkey = "bf16" if a.dtype == "bfloat16" else "fp32"
    pts = {}
    short = max(8, a.steps // 2), max(2, a.warmup // 2)
    for B in points:
        say(f"decode at batch {B}")
        rate, sec = decode_rate(B, *short)
        pts[f"decode_b{B}"] = round(rate, 1)
        pts[f"decode_b{B}_hbm_frac"] = round(hbm_frac(B, a.context, short[0], sec), 4)
    for c in contexts:
        for B in sorted({a.batch, 64} & set([a.batch] + points)):
            say(f"decode at batch {B}, context {c}")
            rate, sec = decode_rate(B, *short, context=c)
            pts[f"decode_b{B}_ctx{c}"] = round(rate, 1)
            pts[f"decode_b{B}_ctx{c}_hbm_frac"] = round(hbm_frac(B, c, short[0], sec), 4)
    for T in [int(t) for t in a.prefill_points.split(",") if t.strip()]:
        if T <= spec_full.max_context and T <= pool:
            say(f"prefill of {T} tokens")
            t = prefill_rate(T, reps=3)
            pts[f"prefill_{T}"] = round(T / t, 1)
            pts[f"prefill_{T}_mfma_frac"] = round(costs.prefill_flops(T) / t / PEAK_FLOPS[dkey], 4)
    if trunk is not None:
        # the reference's "plain" decode runs no prediction heads; the same here, for comparison with its numbers
        say(f"decode at batch {a.batch} without the prediction heads")
        pts[f"decode_b{a.batch}_trunk_only"] = round(decode_rate(a.batch, a.steps, a.warmup, trunk)[0], 1)
    # the same decode at the headline batch through the scheduler: admission, planning, sampling with the reference's
    # options (server.py:515-516), finishing
    say(f"decode at batch {a.batch} through the scheduler")
    pts[f"decode_b{a.batch}_scheduler"] = round(scheduler_decode_rate(engine, a, gen), 1)
    del engine, trunk
    if a.serve_point and a.new_tokens + 130 < min(spec_full.max_context, 8192):
        # whole requests through the scheduler (the serve workload above), so that the record carries it
        say("serve workload")
        torch.cuda.empty_cache()
        line = scheduler_workload(a, cfg, layers_full, tensors, heads, page, say, workload="serve")
        pts["serve_tok_s"] = line["value"]
        pts["serve_floor_frac"] = line["roofline"]["frac"]
    line = {
        "metric": f"decode tok/s at batch {a.batch} ({a.size}, {dkey}); prefill tok/s at {a.prefill_tokens:,} tokens",
        "value": round(value, 1), "unit": "tok/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(sec_per_step * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        # against the reference's figure only where the run is the reference's case: whole model, its size and batch
        "vs_baseline": (round(value / REFERENCE_B8_TOKS, 2)
                        if (a.batch == 8 and a.size == "0.9B" and sizes["n_layers"] == layers_full) else None),
        "dtype": dkey, "data": "synthetic: random weights N(0,0.02), uniform random token ids",
        "config": {
            "model": a.size, "global_batch": a.batch, "seq_len": a.context, "parallelism": "single-gpu",
            **sizes, "n_layers_full": layers_full,
            # the heads' blocks run in every timed step; their logits are not asked for (drafts are not used)
            "mtp_head_logits": False, "max_context": spec_full.max_context, "page_size": page, "sampling": "greedy",
        },
        "prefill": {"value": round(a.prefill_tokens / pt, 1), "tokens": a.prefill_tokens, "ms": round(pt * 1e3, 3),
                    "frac": round(costs.prefill_flops(a.prefill_tokens) / pt / PEAK_FLOPS[dkey], 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_GBS, 4)},
        "points": pts,
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())

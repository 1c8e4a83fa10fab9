#!/usr/bin/env python3
"""Decode and prefill throughput of the engine on one MI355X, with random weights.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--size 0.9B] [--batch 8] [--context 4096]

A step is one decode step: every live request advances by one token through the whole model (trunk, the
prediction heads unless --trunk-only, output table, sampling, read-back of the tokens). One JSON line is
printed: decoded tokens a second at the given batch, the prefill of 2,048 tokens, the decode step's
bandwidth against the HBM peak, and decode at batch 1 and 64.
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


def matmul_params(cfg, heads: bool):
    """Matrix weights a step reads once (elements), and the same without the output table."""
    D, F = cfg.d_model, cfg.ffn_hidden
    kvw = 2 * cfg.n_kv_heads * cfg.head_dim
    block = D * D + D * kvw + D * D + 3 * D * F
    n = cfg.n_layers * block
    if heads:
        n += cfg.mtp_heads * (block + 2 * D * D)
    table = cfg.vocab_size * D
    return n + table, n


def kv_bytes_per_token(cfg, heads: bool, elem: int):
    planes = cfg.n_layers + (cfg.mtp_heads if heads else 0)
    return planes * 2 * cfg.n_kv_heads * cfg.head_dim * elem


def prefill_flops(cfg, T: int, heads: bool):
    with_table, without = matmul_params(cfg, heads)
    linear = 2.0 * without * T + 2.0 * cfg.vocab_size * cfg.d_model      # the output table runs for one row
    planes = cfg.n_layers + (cfg.mtp_heads if heads else 0)
    attention = planes * 4.0 * cfg.n_heads * cfg.head_dim * (T * (T + 1) / 2)
    return linear + attention


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
    ap.add_argument("--points", default="1,64", help="other batch sizes to measure, comma separated ('' for none)")
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--no-trunk-point", dest="trunk_point", action="store_false",
                    help="skip the extra decode measurement without the prediction heads")
    ap.add_argument("--seed", type=int, default=0)
    a = ap.parse_args()
    if a.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {a.gpus} is not supported")
        return 2

    import dataclasses

    import torch

    from tiny_inference_server_amd.__main__ import size_config
    from tiny_inference_server_amd.engine import Engine
    from tiny_inference_server_amd.weights import random_tensors

    def say(what):
        # progress on stderr, flushed: names the phase a run was in if it ends without its line
        print(f"[bench] {what}", file=sys.stderr, flush=True)

    cfg_full = size_config(a.size)
    cfg = cfg_full
    if a.layers and a.layers != cfg_full.n_layers:
        cfg = dataclasses.replace(cfg_full, n_layers=a.layers)
    heads = cfg.mtp_heads > 0 and not a.trunk_only
    dev = "cuda:0"
    torch.cuda.set_device(0)
    tensors = random_tensors(cfg, a.seed, dtype=a.dtype, device=dev)
    points = [int(p) for p in a.points.split(",") if p.strip()]
    max_b = max([a.batch] + points)
    page = 16
    engine = Engine(config=cfg, tensors=tensors, dtype=a.dtype, page_size=page,
                    max_tokens=max_b * (a.context + page), max_requests=max_b, device=dev, run_heads=heads)
    trunk = None
    if heads and a.trunk_point:
        trunk = Engine(config=cfg, tensors=tensors, dtype=a.dtype, page_size=page,
                       max_tokens=a.batch * (a.context + page), max_requests=a.batch, device=dev, run_heads=False)
    del tensors
    vocab = cfg.vocab_size
    gen = torch.Generator().manual_seed(a.seed)

    def decode_rate(B: int, steps: int, warmup: int, engine=engine):
        """Tokens a second and seconds per step of `steps` decode steps at batch B near the context length."""
        start_len = a.context - steps - warmup - 1
        rids = [f"b{B}_{i}" for i in range(B)]
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

    say(f"{a.size}, {cfg.n_layers} layers, {a.dtype}: decode at batch {a.batch}, context {a.context}")
    value, sec_per_step = decode_rate(a.batch, a.steps, a.warmup)
    elem = 2 if a.dtype == "bfloat16" else 4
    with_table, _ = matmul_params(cfg, heads)
    step_bytes = with_table * elem + a.batch * (a.context - a.steps // 2) * kv_bytes_per_token(cfg, heads, elem)
    achieved = step_bytes / sec_per_step / 1e9
    say(f"prefill of {a.prefill_tokens} tokens")
    pt = prefill_rate(a.prefill_tokens)
    dkey = "bf16" if a.dtype == "bfloat16" else "fp32"
    pf = prefill_flops(cfg, a.prefill_tokens, heads)
    pts = {}
    for B in points:
        say(f"decode at batch {B}")
        pts[f"decode_b{B}"] = round(decode_rate(B, max(8, a.steps // 2), max(2, a.warmup // 2))[0], 1)
    if trunk is not None:
        # the reference's "plain" decode runs no prediction heads; the same here, for comparison with its numbers
        say(f"decode at batch {a.batch} without the prediction heads")
        pts[f"decode_b{a.batch}_trunk_only"] = round(decode_rate(a.batch, a.steps, a.warmup, trunk)[0], 1)
    line = {
        "metric": f"decode tok/s at batch {a.batch} ({a.size}, {dkey}); prefill tok/s at {a.prefill_tokens:,} tokens",
        "value": round(value, 1), "unit": "tok/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(sec_per_step * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        # against the reference's figure only where the run is the reference's case: whole model, its size and batch
        "vs_baseline": (round(value / REFERENCE_B8_TOKS, 2)
                        if (a.batch == 8 and a.size == "0.9B" and cfg.n_layers == cfg_full.n_layers) else None),
        "dtype": dkey, "data": "synthetic: random weights N(0,0.02), uniform random token ids",
        "config": {
            "model": a.size, "global_batch": a.batch, "seq_len": a.context, "parallelism": "single-gpu",
            "n_layers": cfg.n_layers, "n_layers_full": cfg_full.n_layers, "d_model": cfg.d_model,
            "n_heads": cfg.n_heads, "n_kv_heads": cfg.n_kv_heads, "head_dim": cfg.head_dim,
            "ffn_hidden": cfg.ffn_hidden, "vocab_size": cfg.vocab_size,
            "mtp_heads_run": cfg.mtp_heads if heads else 0,
            "tie_embeddings": cfg.tie_embeddings, "rope_base": cfg.rope_base, "page_size": page,
            "sampling": "greedy",
        },
        "prefill": {"value": round(a.prefill_tokens / pt, 1), "tokens": a.prefill_tokens, "ms": round(pt * 1e3, 3),
                    "frac": round(pf / pt / PEAK_FLOPS[dkey], 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_GBS, 4)},
        "points": pts,
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())

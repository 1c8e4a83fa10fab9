"""Trace replay: feed given token ids through the engine's step function, step by step, and write logits.

It samples nothing and has no model code of its own: it builds the same Engine that generation uses and
calls its step function. Steps arrive as JSON lines on standard input:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

For a step in which something is wanted, `<out>/<step>.f32` holds the logits at the wanted places in the
order of the entries and of `want`, little-endian 32-bit floats, [wanted, vocab]. With `heads`, the
prediction heads' logits at the same rows go to `<out>/<step>.head<i>.f32` (NaN where a head has no row
yet). After every step the line `done <step>` is printed and flushed.
"""
from __future__ import annotations

import json
import os
import sys
from typing import IO, Optional

from .engine import Engine


def replay(model_dir: str, dtype: str, out_dir: str, max_tokens: int, lines: IO[str], out: IO[str] = sys.stdout,
           page_size: int = 16, max_requests: int = 8, heads: bool = False, device: str = "cuda:0",
           ops=None) -> int:
    os.makedirs(out_dir, exist_ok=True)
    print(f"[trace_run] loading {model_dir} as {dtype}", file=sys.stderr, flush=True)
    # max_tokens counts every live request rounded up to a multiple of 64. With a page size that divides 64 that is
    # whole pages already; with any other, a request's last page may reach past its rounded count by less than one
    # page, so the pool gets one page more per request that can be live.
    n_pages = -(-max_tokens // page_size) + (0 if 64 % page_size == 0 else max_requests)
    engine = Engine(model_dir, dtype=dtype, page_size=page_size, n_pages=n_pages, max_requests=max_requests,
                    device=device, ops=ops)
    print(f"[trace_run] ready: {engine.total_pages()} pages of {page_size} tokens", file=sys.stderr, flush=True)
    for line in lines:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step_id = rec["step"]
        entries = [(e["id"], e["tokens"], e.get("want", [])) for e in rec.get("entries", [])]
        if entries:
            res = engine.step(entries, heads=heads)
            if res.logits.shape[0]:
                arr = res.logits.detach().to("cpu").numpy().astype("<f4", copy=False)
                arr.tofile(os.path.join(out_dir, f"{step_id}.f32"))
                if heads and res.head_logits:
                    for i, hl in enumerate(res.head_logits):
                        hl.detach().to("cpu").numpy().astype("<f4", copy=False).tofile(
                            os.path.join(out_dir, f"{step_id}.head{i}.f32"))
        for rid in rec.get("end", []):
            if rid in engine.requests:
                engine.close(rid)
        print(f"done {step_id}", file=out, flush=True)
    return 0


def main(argv: Optional[list] = None) -> int:
    import argparse
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    ap.add_argument("--out", required=True, help="folder for the <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens that live requests hold at any time; the cache pool is made for this many")
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--max-requests", type=int, default=8)
    ap.add_argument("--heads", action="store_true", help="also write the prediction heads' logits")
    ap.add_argument("--device", default="cuda:0")
    a = ap.parse_args(argv)
    if a.page_size < 1:
        ap.error("--page-size must be at least 1")
    return replay(a.model, a.dtype, a.out, a.max_tokens, sys.stdin, sys.stdout, a.page_size, a.max_requests,
                  a.heads, a.device)

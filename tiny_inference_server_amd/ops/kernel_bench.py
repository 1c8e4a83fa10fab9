"""Times one kernel alone on synthetic operands, for profiling runs and for tuning.

    python -m tiny_inference_server_amd.ops.kernel_bench attention --segments 0:2048
    python -m tiny_inference_server_amd.ops.kernel_bench attention --segments 4095:1x8
    python -m tiny_inference_server_amd.ops.kernel_bench attention --segments 0:2048 --no-tiles
    python -m tiny_inference_server_amd.ops.kernel_bench product --rows 8 --out 8192 --in 1536 --kind norm+gate

A segment is `first position:rows`, `xN` repeats it for N requests; `4095:1x8` is a decode step of 8 requests at
context 4096, `0:2048` a prompt of 2,048 tokens, `4095:1x8,1000:256` a mixed step. Long portions go to the
workgroup (tile) kernel where the engine would send them; `--tiles` sends them there however little work they are,
`--no-tiles` keeps every row with the one-wave kernel. The kernel is captured into a
graph of `--reps` launches and the graph is timed, so host launch cost stays out. A kernel alone runs on warm caches:
decisions about decode kernels are taken on whole decode steps (bench.py), this is for counters and first looks.
"""
from __future__ import annotations

import argparse
import sys
from types import SimpleNamespace

import torch


def graph_time(fn, reps: int) -> float:
    """Microseconds per call of `fn`, median of seven replays of a graph that holds `reps` calls."""
    fn()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for _ in range(reps):
            fn()
    g.replay()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    times = []
    for _ in range(7):
        a.record()
        g.replay()
        b.record()
        torch.cuda.synchronize()
        times.append(a.elapsed_time(b) * 1000 / reps)
    return sorted(times)[3]


def parse_segments(text: str):
    segs = []
    for part in text.split(","):
        body, _, times = part.partition("x")
        first, _, rows = body.partition(":")
        segs += [(int(first), int(rows))] * (int(times) if times else 1)
    return segs


def attention_case(ops, a):
    from .hip_ops import attention_items, decode_items, planned_list_pays, tile_columns, uneven_lengths
    nh, kvh, hd, ps = a.heads, a.kv_heads, a.head_dim, a.page_size
    segs = parse_segments(a.segments)
    pages = [-(-(p0 + n) // ps) for p0, n in segs]
    plane = torch.randn(sum(pages) + 4, 2, kvh, ps, hd, device=ops.device).to(torch.bfloat16)
    tables = torch.zeros(len(segs), max(pages), dtype=torch.int32)
    positions, row_seq, seq_rows, nxt = [], [], [], 0
    for i, ((p0, n), k) in enumerate(zip(segs, pages)):
        tables[i, :k] = torch.arange(nxt, nxt + k)
        nxt += k
        seq_rows.append((len(positions), p0, n))
        positions += list(range(p0, p0 + n))
        row_seq += [i] * n
    rows = len(positions)
    q = torch.randn(rows, nh * hd, device=ops.device).to(torch.bfloat16)
    batch = SimpleNamespace(positions=torch.tensor(positions, dtype=torch.int32, device=ops.device),
                            row_seq=torch.tensor(row_seq, dtype=torch.int32, device=ops.device),
                            block_tables={"g": tables.to(ops.device)}, max_kv_len=max(p0 + n for p0, n in segs),
                            extras={}, n_rows=rows, max_seq_rows=max(n for _, n in segs), seq_rows=seq_rows)
    # --no-tiles: what the one-wave kernel alone makes of the same rows; --tiles: tiles however little work there is
    import numpy as np
    if ((uneven_lengths(seq_rows) and planned_list_pays(len(seq_rows), kvh)) or a.planned) and not a.same_splits:
        # decoded tokens of requests that differ widely in length: splits planned request by request, as the engine does
        entries, most = decode_items(seq_rows, nh, kvh, hd)
        batch.extras[("attention_decode_items", nh // kvh, tile_columns(hd), kvh, 0)] = (
            torch.from_numpy(entries).reshape(-1).to(ops.device), len(entries), most)
    else:
        from .hip_ops import planned_beside_tiles
        nb, items, tiles, steps = attention_items(seq_rows, nh // kvh, 0 if a.no_tiles else tile_columns(hd),
                                                  0 if a.tiles else kvh)
        beside = None if a.same_splits else planned_beside_tiles(seq_rows, items, tiles, steps, nh, kvh, hd, 0, ops.units)
        if beside is not None:      # decoded tokens of uneven lengths beside a portion's tiles: as the engine plans them
            both = np.concatenate((beside[0].reshape(-1), tiles.reshape(-1)))
            plan = (torch.from_numpy(np.ascontiguousarray(both)).to(ops.device), len(beside[0]), 1, len(tiles), steps, beside[1])
        else:
            both = torch.from_numpy(np.ascontiguousarray(np.concatenate((items, tiles)))).reshape(-1).to(ops.device)
            plan = (both, len(items), nb, len(tiles), steps, 0)
        batch.extras[("attention_items", nh // kvh, tile_columns(hd), kvh, 0)] = plan
    us = graph_time(lambda: ops.paged_attention(q, plane, batch, "g", nh, kvh, hd), a.reps)
    kv_bytes = sum(p0 + n for p0, n in segs) * kvh * hd * 2 * 2
    flops = sum(4 * nh * hd * (n * p0 + n * (n + 1) / 2) for p0, n in segs)
    print(f"attention {a.segments}: {us:.1f} us; keys and values {kv_bytes / 1e6:.1f} MB -> {kv_bytes / us / 1e6:.2f} TB/s; "
          f"{flops / us / 1e6:.1f} TFLOP/s")


def product_case(ops, a):
    m, n, k = a.rows, a.out, a.inner
    x = torch.randn(m, k, device=ops.device).to(torch.bfloat16)
    # --copies: the launches take their weights from that many matrices in turn, so that with enough of them (their
    # bytes beyond the 256 MB of the memory-side cache) every launch streams its weights from HBM as in a decode step
    ws = [(torch.randn(n, k, device=ops.device) * k ** -0.5).to(torch.bfloat16) for _ in range(max(1, a.copies))]
    res = torch.randn(m, n, device=ops.device).to(torch.bfloat16)
    rms = (torch.ones(k, device=ops.device), 1e-6)
    turn = [0]

    def w():
        turn[0] += 1
        return ws[turn[0] % len(ws)]
    kinds = {"plain": lambda: ops.linear(x, w()), "residual": lambda: ops.linear(x, w(), residual=res),
             "norm": lambda: ops.linear(x, w(), rms=rms), "norm+gate": lambda: ops.linear_swiglu(x, w(), rms=rms),
             "logits": lambda: ops.linear(x, w(), out_dtype=torch.float32)}
    if a.few_rows:
        ops.few_rows = a.few_rows
    if a.staged:
        ops.gemm_skinny.cdll.tis_gemm_skinny_staged_stages(int(a.staged))
    if a.staged_always:
        ops.gemm_skinny.cdll.tis_gemm_skinny_staged_always(1)
    us = graph_time(kinds[a.kind], a.reps)
    print(f"product {a.kind} rows {m} out {n} in {k}: {us:.2f} us; weights {n * k * 2 / 1e6:.1f} MB -> "
          f"{n * k * 2 / us / 1e6:.2f} TB/s; {2 * m * n * k / us / 1e6:.1f} TFLOP/s")


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="python -m tiny_inference_server_amd.ops.kernel_bench", description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    sub = ap.add_subparsers(dest="what", required=True)
    at = sub.add_parser("attention")
    at.add_argument("--segments", default="4095:1x8")
    at.add_argument("--heads", type=int, default=12)
    at.add_argument("--kv-heads", type=int, default=3)
    at.add_argument("--head-dim", type=int, default=128)
    at.add_argument("--page-size", type=int, default=16)
    at.add_argument("--no-tiles", action="store_true", help="long portions too go to the one-wave kernel")
    at.add_argument("--tiles", action="store_true", help="long portions go to the workgroup kernel however few they are")
    at.add_argument("--planned", action="store_true",
                    help="decoded tokens: splits planned request by request also where the lengths are alike")
    at.add_argument("--same-splits", action="store_true",
                    help="decoded tokens: every request gets the same number of splits, however their lengths differ")
    pr = sub.add_parser("product")
    pr.add_argument("--rows", type=int, default=8)
    pr.add_argument("--out", type=int, default=8192)
    pr.add_argument("--in", dest="inner", type=int, default=1536)
    pr.add_argument("--kind", choices=["plain", "residual", "norm", "norm+gate", "logits"], default="plain")
    pr.add_argument("--copies", type=int, default=1, help="weight matrices that the launches take in turn")
    pr.add_argument("--staged", default="", help="LDS stages of the few-row kernel for 17 rows and more: 2 or 4 (default: its own choice)")
    pr.add_argument("--staged-always", action="store_true", help="that kernel also for up to 8 rows of narrow matrices")
    pr.add_argument("--few-rows", type=int, default=0, help="the row count up to which the few-row kernel is used (0: as built)")
    for p in (at, pr):
        p.add_argument("--reps", type=int, default=20)
        p.add_argument("--device", default="cuda:0")
    a = ap.parse_args(argv)
    from .hip_ops import HipOps
    ops = HipOps(a.device, torch.bfloat16)
    (attention_case if a.what == "attention" else product_case)(ops, a)
    return 0


if __name__ == "__main__":
    sys.exit(main())

"""Command line: run prompts through the scheduler and print the generated token ids and tokens a second.

The reference's `python server.py` has no flags: its settings are constants at the top of the file
(server.py:12-19) and arguments of Request and Scheduler (server.py:79, 106). The options here carry those
names: --pool-bytes, --tokens-per-block, --max-batch, --device, --plan; --max-new-tokens, --temperature,
--top-k, --top-p, --rep-penalty, with the reference's run defaults (server.py:515-516). Prompts are token ids,
since this build has no tokenizer: given with --prompt-ids, or drawn at random with --prompt-len/--num-prompts.
"""
from __future__ import annotations

import argparse
import os
import random
import sys
import tempfile
import time

PRESETS = os.path.join(os.path.dirname(os.path.abspath(__file__)), "config", "presets")


def preset_names():
    return sorted(f[:-5] for f in os.listdir(PRESETS) if f.endswith(".json"))


def size_config(name: str):
    """The configuration of a named size: a config.json under config/presets/."""
    import json

    from . import architectures  # noqa: F401
    from .config import config_from_dict
    with open(os.path.join(PRESETS, name + ".json")) as f:
        return config_from_dict(json.load(f))


def parse_bytes(text: str) -> int:
    t = text.strip().lower()
    for suffix, mul in (("gib", 1 << 30), ("gb", 10 ** 9), ("mib", 1 << 20), ("mb", 10 ** 6), ("g", 1 << 30), ("m", 1 << 20)):
        if t.endswith(suffix):
            return int(float(t[:-len(suffix)]) * mul)
    return int(t)


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="python -m tiny_inference_server_amd", description=__doc__.split("\n\n")[0])
    src = ap.add_mutually_exclusive_group(required=True)
    src.add_argument("--model", help="model folder with config.json and model.safetensors")
    src.add_argument("--random", choices=preset_names(), help="random weights of a named size")
    ap.add_argument("--write-model", metavar="DIR", help="with --random: write the model folder there and exit")
    ap.add_argument("--seed", type=int, default=0, help="seed of the random weights, the prompts and the sampling")
    ap.add_argument("--prompt-ids", action="append", default=[], metavar="IDS", help="comma-separated token ids; repeatable")
    ap.add_argument("--prompt-len", type=int, default=10)
    ap.add_argument("--num-prompts", type=int, default=10)
    ap.add_argument("--max-new-tokens", type=int, default=200)
    ap.add_argument("--temperature", type=float, default=0.9)
    ap.add_argument("--top-k", type=int, default=50)
    ap.add_argument("--top-p", type=float, default=0.95)
    ap.add_argument("--rep-penalty", type=float, default=1.1)
    ap.add_argument("--greedy", action="store_true", help="arg-max decoding (temperature 0)")
    ap.add_argument("--ignore-eos", action="store_true")
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    ap.add_argument("--device", default="cuda:0")
    ap.add_argument("--max-batch", type=int, default=8)
    ap.add_argument("--pool-bytes", default="4GiB", help="memory of the page pool")
    ap.add_argument("--tokens-per-block", type=int, default=16)
    ap.add_argument("--token-budget", type=int, default=2048, help="most tokens one step runs")
    ap.add_argument("--plan", choices=["final", "cur"], default="final")
    ap.add_argument("--static", default=None, metavar="MODE",
                    help="take a request's pages at admission: 'ctx' (whole context), 'req' (prompt + new tokens) or a "
                         "number of tokens; default: pages on demand")
    ap.add_argument("--heads", action="store_true",
                    help="also run the multi-token-prediction heads at every step (their drafts are not used)")
    a = ap.parse_args(argv)

    from .config import ARCHITECTURES, load_config
    from .engine import Engine
    from .engine.generate import generate
    from .weights import write_random_model

    tmp = None
    if a.random:
        cfg = size_config(a.random)
        if a.write_model:
            write_random_model(cfg, a.seed, a.write_model)
            print(f"wrote {a.write_model}")
            return 0
        tmp = tempfile.TemporaryDirectory(prefix="tis_amd_model_")
        model_dir = write_random_model(cfg, a.seed, tmp.name)
    else:
        model_dir = a.model
        cfg = load_config(model_dir)
    if a.prompt_ids:
        prompts = [[int(t) for t in p.replace(" ", "").split(",") if t] for p in a.prompt_ids]
    else:
        rng = random.Random(a.seed)
        vocab = ARCHITECTURES.get(cfg.architecture).build_spec(cfg).vocab_size
        prompts = [[rng.randrange(vocab) for _ in range(a.prompt_len)] for _ in range(a.num_prompts)]

    # as many pages as the bytes hold, whatever the model's parts keep in a page (reference block_table.py:34-38)
    engine = Engine(model_dir, dtype=a.dtype, page_size=a.tokens_per_block, pool_bytes=parse_bytes(a.pool_bytes),
                    max_requests=a.max_batch, device=a.device, run_heads=a.heads)
    if engine.cache.groups:
        print(f"POOL: {engine.total_pages()} blocks of {a.tokens_per_block} tokens", file=sys.stderr)
    import torch
    t0 = time.time()
    outs, sched = generate(engine, prompts, max_new_tokens=a.max_new_tokens,
                           temperature=0.0 if a.greedy else a.temperature, top_k=0 if a.greedy else a.top_k,
                           top_p=0.0 if a.greedy else a.top_p, rep_penalty=1.0 if a.greedy else a.rep_penalty,
                           seed=a.seed, ignore_eos=a.ignore_eos, max_batch=a.max_batch, token_budget=a.token_budget,
                           plan=a.plan, static=(int(a.static) if a.static and a.static.isdigit() else a.static),
                           return_scheduler=True)
    torch.cuda.synchronize()
    dt = time.time() - t0
    total = sum(len(o) for o in outs)
    print(f"\n{total} tokens in {dt:.1f}s ({total / dt:.1f} tok/s), {sched.steps} steps, {sched.preempts} preemptions\n")
    for p, o in zip(prompts, outs):
        print("=" * 100)
        print("PROMPT:", " ".join(map(str, p)))
        print("OUTPUT:", " ".join(map(str, o)))
    if tmp is not None:
        tmp.cleanup()
    return 0


if __name__ == "__main__":
    sys.exit(main())

"""Generation through the entry points on the GPU, and the replay program as a user runs it."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import helpers as H
import plain_model as pm
from tiny_inference_server_amd.engine.generate import generate
from tiny_inference_server_amd.sampling import SamplingParams, uniform_for

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_equals_plain(name):
    """Two tiny workloads: 3 prompts of 5/17/33 tokens (A) and 4 of 1/9/24/40 tokens (B), 16 greedy tokens each."""
    folder = H.model_folder(name, "float32")
    cfg, w = pm.read_model_folder(folder)
    lens = [5, 17, 33] if name == "A" else [1, 9, 24, 40]
    prompts = [H.random_ids(cfg["vocab"], n, 90 + i) for i, n in enumerate(lens)]
    want = [pm.greedy_generate(p, 16, w, cfg) for p in prompts]
    ps = H.TINY[name]["page_size"]
    assert generate(folder, prompts, max_new_tokens=16, temperature=0.0, dtype="float32", tokens_per_block=ps) == want
    # portions under a small token budget, few pages, preemption allowed: the same tokens
    got, s = generate(folder, prompts, max_new_tokens=16, temperature=0.0, dtype="float32", tokens_per_block=ps,
                      max_batch=2, token_budget=9, plan="cur", pool_tokens=5 * 16, return_scheduler=True)
    assert got == want and s.engine.free_pages() == s.engine.total_pages()


def test_bfloat16_generation_follows_the_plain_choice_where_it_is_clear():
    """In bfloat16 an arg-max may flip where two logits are close; where the plain model's margin is wide it must not."""
    folder = H.model_folder("D", "bfloat16")
    cfg, w = pm.read_model_folder(folder)
    prompts = [H.random_ids(cfg["vocab"], n, 95 + i) for i, n in enumerate([12, 30])]
    got = generate(folder, prompts, max_new_tokens=12, temperature=0.0, dtype="bfloat16")
    for p, g in zip(prompts, got):
        ids = list(p)
        for t in g:
            lg = pm.logits_of(pm.trunk_hidden(ids, w, cfg)[-1:], w, cfg)[0]
            top2 = torch.topk(lg, 2).values
            if (top2[0] - top2[1]).item() > 0.1:
                assert t == int(lg.argmax())
            ids.append(t)


def test_bfloat16_scheduler_with_heads_and_preemption():
    """The scheduler on the GPU in bfloat16 with the prediction heads run at every step, as many slots as requests,
    a pool that forces preemption under plan "cur", and prompts cut by a small token budget (the reference's own
    model-level check of its scheduler: test_server.py:66-118). Tokens are compared with the plain model's choice
    wherever that choice is clear (bfloat16 may flip an arg-max between two close logits)."""
    folder = H.model_folder("D", "bfloat16")
    cfg, w = pm.read_model_folder(folder)
    lens, new = [30, 12, 21, 9, 17], [20, 6, 12, 16, 8]
    prompts = [H.random_ids(cfg["vocab"], n, 140 + i) for i, n in enumerate(lens)]
    params = [SamplingParams(max_new_tokens=k, temperature=0.0, ignore_eos=True) for k in new]
    got, s = generate(folder, prompts, params=params, dtype="bfloat16", max_batch=3, token_budget=24, plan="cur",
                      pool_tokens=96, run_heads=True, return_scheduler=True)
    assert s.preempts > 0 and s.engine.graph_replays > 0
    assert len(s.engine.model.spec.stages) == 3          # the heads did run
    checked = 0
    for p, g, k in zip(prompts, got, new):
        assert len(g) == k
        ids = list(p)
        for t in g:
            lg = pm.logits_of(pm.trunk_hidden(ids, w, cfg)[-1:], w, cfg)[0]
            top2 = torch.topk(lg, 2).values
            if (top2[0] - top2[1]).item() > 0.1:
                assert t == int(lg.argmax())
                checked += 1
            ids.append(t)
    assert checked >= sum(new) // 2
    s.engine.cache.check()
    assert s.engine.free_pages() == s.engine.total_pages()


def test_scheduler_at_the_headline_geometry_with_fourteen_sampled_requests_on_a_pool_of_nan():
    """Where the captured steps' filler lines, per-request attention splits, preemption, the prediction heads and the
    sampling kernel's penalty tables meet: 14 requests at the headline model's layer sizes (12 query heads of 128 over
    3, width 1536) in bfloat16, heads run at every step, plan "cur" on a pool that cannot hold them all, sampled with a
    temperature and a repetition penalty, every page filled with NaN beforehand (reference's model-level check of its
    scheduler: test_server.py:66-118). Steps of 9 to 14 decoded tokens are filled up to 16 lines with the cache
    manager's own request and replayed from captured graphs; every token lies where the reference's sampling rule
    puts it on the plain model's logits, up to what bfloat16 moves the cumulative distribution by."""
    from tiny_inference_server_amd.engine import Engine
    from tiny_inference_server_amd.engine.scheduler import Request, Scheduler
    name, n_req = "E", 14
    folder = H.model_folder(name, "bfloat16")
    prompts, params = H.sampled_workload(name, n_req, seed=300)
    eng = Engine(folder, dtype="bfloat16", page_size=16, max_tokens=47 * 16, max_requests=n_req, run_heads=True)
    H.fill_cache_with_nan(eng)
    steps = H.watch_decode_steps(eng)
    s = Scheduler(eng, max_batch=n_req, token_budget=96, plan="cur")
    reqs = [Request(p, sp) for p, sp in zip(prompts, params)]
    for r in reqs:
        s.submit(r)
    s.run()
    assert s.preempts > 0 and s.replays > 0 and eng.graph_replays > 0
    assert any(n > 8 and n % 8 and replayed for n, replayed in steps), steps       # a filled-up shape was replayed
    assert s.peak_running > 8
    checked, equal = H.check_sampled_tokens(folder, prompts, params, [r.out_ids() for r in reqs], slack=0.08)
    assert checked == sum(sp.max_new_tokens for sp in params) and equal >= checked // 3, (checked, equal)
    eng.cache.check()
    assert eng.free_pages() == eng.total_pages() and eng.cache.n_live == 0


@pytest.mark.parametrize("seed", range(12))
def test_scheduler_on_drawn_configurations_with_drawn_sampling(seed):
    """Every size of the model drawn at random, then the scheduler's own knobs (requests, slots, token budget, plan,
    a pool from too small for all to ample, heads run or not) and each request's sampling (arg-max, temperatures,
    top-k, top-p, repetition penalty) drawn too, in 32-bit on a pool full of NaN: every sampled token is the plain
    rule's draw on the plain model's logits (server.py:22-50) up to rounding at a boundary of the cumulative
    distribution, every arg-max token the plain arg-max where that is clear, and nothing is left in the cache."""
    import random
    from test_engine_schedules import drawn_configuration
    from tiny_inference_server_amd.engine import Engine
    from tiny_inference_server_amd.engine.scheduler import Request, Scheduler
    name = f"scheduled{seed}"
    rng, H.TINY[name] = drawn_configuration(seed + 900)
    cfg, page = H.TINY[name]["cfg"], H.TINY[name]["page_size"]
    n_req = rng.choice([2, 4, 6, 10, 14])
    prompts = [H.random_ids(cfg.vocab_size, rng.randint(1, 60), seed * 50 + i) for i in range(n_req)]
    params = [SamplingParams(max_new_tokens=rng.randint(3, 20), temperature=rng.choice([0.0, 0.3, 0.8, 1.0]),
                             top_k=rng.choice([0, 0, 5, 40]), top_p=rng.choice([1.0, 1.0, 0.9, 0.5]),
                             rep_penalty=rng.choice([1.0, 1.3]), seed=seed * 10 + i, ignore_eos=True) for i in range(n_req)]
    sizes = [len(p) + sp.max_new_tokens for p, sp in zip(prompts, params)]
    pool = max(-(-max(sizes) // page) * page + page, int(sum(sizes) * rng.choice([0.4, 0.7, 1.2])) // page * page)
    plan, heads, max_batch = rng.choice(["cur", "final"]), rng.random() < 0.5, rng.choice([2, 4, n_req])
    budget = max(rng.choice([8, 24, 64, 256]), max_batch)
    folder = H.model_folder(name, "float32")
    eng = Engine(folder, dtype="float32", page_size=page, max_tokens=pool, max_requests=max_batch, run_heads=heads)
    H.fill_cache_with_nan(eng)
    s = Scheduler(eng, max_batch=max_batch, token_budget=budget, plan=plan)
    reqs = [Request(p, sp) for p, sp in zip(prompts, params)]
    for r in reqs:
        s.submit(r)
    s.run()
    sampled = [i for i, sp in enumerate(params) if sp.temperature > 0.0]
    H.check_sampled_tokens(folder, [prompts[i] for i in sampled], [params[i] for i in sampled],
                           [reqs[i].out_ids() for i in sampled], slack=1e-4)
    model_cfg, w = pm.read_model_folder(folder)
    for i, sp in enumerate(params):
        out = reqs[i].out_ids()
        assert len(out) == sp.max_new_tokens
        if sp.temperature > 0.0 or sp.rep_penalty != 1.0:
            continue
        ids = list(prompts[i])
        for t in out:
            lg = pm.logits_of(pm.trunk_hidden(ids, w, model_cfg)[-1:], w, model_cfg)[0]
            top2 = torch.topk(lg, 2).values
            assert t == int(lg.argmax()) or (top2[0] - top2[1]).item() < 1e-3
            ids.append(t)
    eng.cache.check()
    assert eng.free_pages() == eng.total_pages() and eng.cache.n_live == 0


def test_temperature_sampling_with_seeded_streams():
    """Tiny B's workload: temperature 0.8, seed 0, mixed chunked prefill and decode; token by token the draw is the
    plain rule's (server.py:22-50) on the plain logits with the request's own uniform number."""
    folder = H.model_folder("B", "float32")
    cfg, w = pm.read_model_folder(folder)
    prompts = [H.random_ids(cfg["vocab"], n, 97 + i) for i, n in enumerate([1, 9, 24, 40])]
    params = [SamplingParams(max_new_tokens=8, temperature=0.8, seed=i) for i in range(4)]
    got = generate(folder, prompts, params=params, dtype="float32", tokens_per_block=8, token_budget=16, max_batch=4)
    for p, sp, g in zip(prompts, params, got):
        ids = list(p)
        for i in range(8):
            lg = pm.logits_of(pm.trunk_hidden(ids, w, cfg)[-1:], w, cfg)[0]
            probs = pm.sampling_probs(lg, sp.temperature)
            u = uniform_for(sp.seed, i)
            c = torch.cumsum(probs, 0)
            want = pm.pick_by_uniform(probs, u)
            # a draw that lands within rounding of a boundary of the cumulative distribution may go either way
            near = (c - u).abs().min().item() < 1e-5
            assert g[i] == want or near, (i, g[i], want)
            ids.append(g[i])


def test_command_line_runs(tmp_path):
    folder = H.model_folder("A", "bfloat16")
    out = subprocess.run([sys.executable, "-m", "tiny_inference_server_amd", "--model", folder, "--prompt-ids", "5,17,3",
                          "--prompt-ids", "9", "--max-new-tokens", "5", "--greedy", "--pool-bytes", "1MiB"],
                         cwd=ROOT, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    lines = [l for l in out.stdout.splitlines() if l.startswith("OUTPUT:")]
    assert len(lines) == 2 and all(len(l.split()) == 6 for l in lines)
    assert "tok/s" in out.stdout


@pytest.mark.parametrize("dtype,tol", [("float32", 2e-5), ("bfloat16", 2e-2)])
def test_replay_program(tmp_path, dtype, tol):
    """bin/trace_run as a subprocess: mixed steps with so few pages that they are used again."""
    name = "C"
    folder = H.model_folder(name, "float32" if dtype == "float32" else "bfloat16")
    vocab = H.TINY[name]["cfg"].vocab_size
    reqs = {f"r{i}": H.random_ids(vocab, n, 70 + i) for i, n in enumerate([40, 64, 30, 70, 12, 50])}
    steps, peak = H.mixed_trace(reqs, max_live=4, seed=8)
    out_dir = tmp_path / "out"
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
                           "--out", str(out_dir), "--max-tokens", str(peak), "--heads"],
                          input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-3000:]
    assert proc.stdout.split() == [w for s in steps for w in ("done", str(s["step"]))]
    fed = {r: 0 for r in reqs}
    worst = 0.0
    scale = max(1.0, max(H.plain_logits(folder, ids)[0].abs().max().item() for ids in reqs.values()))
    for s in steps:
        wanted = sum(len(e["want"]) for e in s["entries"])
        arr = np.fromfile(out_dir / f"{s['step']}.f32", dtype="<f4").reshape(wanted, vocab)
        h0 = np.fromfile(out_dir / f"{s['step']}.head0.f32", dtype="<f4").reshape(wanted, vocab)
        row = 0
        for e in s["entries"]:
            main, heads = H.plain_logits(folder, reqs[e["id"]])
            for i in e["want"]:
                p = fed[e["id"]] + i
                worst = max(worst, np.abs(arr[row] - main[p].numpy()).max())
                if p - 1 >= 0:
                    worst = max(worst, np.abs(h0[row] - heads[0][p - 1].numpy()).max())
                else:
                    assert np.isnan(h0[row]).all()
                row += 1
            fed[e["id"]] += len(e["tokens"])
    assert worst <= tol * scale


@pytest.mark.parametrize("args,keys", [
    (["--context", "200", "--steps", "4", "--warmup", "2", "--points", "1", "--prefill-tokens", "64"],
     ("prefill", "roofline", "points")),
    (["--workload", "serve", "--requests", "6", "--new-tokens", "5", "--prefill-tokens", "64"], ("roofline", "detail")),
    (["--workload", "mixed", "--requests", "3", "--steps", "6", "--warmup", "2", "--prefill-tokens", "64"],
     ("roofline", "detail")),
])
def test_bench_modes_run_at_the_tiny_size(args, keys):
    """bench.py's decode line and its two scheduler workloads, at the tiny preset: one JSON line each, with the
    contract's fields, a flat `config` of at most 20 keys, and for more than one GPU a refusal with exit code 2."""
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--size", "tiny"] + args,
                          capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-3000:]
    lines = [l for l in proc.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for k in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
              "vs_baseline", "dtype", "data", "config") + keys:
        assert k in d, k
    assert d["value"] > 0 and d["n_gpus"] == 1 and d["unit"] == "tok/s"
    assert len(d["config"]) <= 20 and all(not isinstance(v, (dict, list)) for v in d["config"].values())
    if "points" in keys:
        assert d["points"]["decode_b1"] > 0 and d["points"]["decode_b8_scheduler"] > 0
    refused = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True,
                             text=True, timeout=60)
    assert refused.returncode == 2 and len(refused.stdout.strip().splitlines()) == 1

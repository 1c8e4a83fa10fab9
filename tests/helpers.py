"""Tiny configurations, model folders in temporary places, traces and their comparison with the plain model."""
from __future__ import annotations

import os
import random
import tempfile
from typing import Dict, List, Sequence, Tuple

import torch

from tiny_inference_server_amd.config import GqaMtpConfig
from tiny_inference_server_amd.weights import write_random_model

import plain_model as pm

# Two tiny configurations that differ in every size and option; C and D add head sizes the fast kernels take.
TINY = {
    "A": dict(cfg=GqaMtpConfig(d_model=64, vocab_size=512, max_context=256, rope_base=10000.0, n_heads=8, n_layers=2,
                               ffn_hidden=176, group_size=4, mtp_heads=1, rms_eps=2e-8, tie_embeddings=True),
              page_size=16, gain_jitter=0.0, seed=11),
    "B": dict(cfg=GqaMtpConfig(d_model=96, vocab_size=1000, max_context=192, rope_base=500000.0, n_heads=3,
                               n_layers=3, ffn_hidden=256, group_size=3, mtp_heads=2, rms_eps=1e-5,
                               tie_embeddings=False),
              page_size=8, gain_jitter=0.1, seed=12),
    "C": dict(cfg=GqaMtpConfig(d_model=192, vocab_size=777, max_context=320, rope_base=1000.0, n_heads=4, n_layers=2,
                               ffn_hidden=200, group_size=2, mtp_heads=1, rms_eps=1e-6, tie_embeddings=True),
              page_size=16, gain_jitter=0.1, seed=13),
    "D": dict(cfg=GqaMtpConfig(d_model=256, vocab_size=515, max_context=640, rope_base=10000.0, n_heads=2, n_layers=2,
                               ffn_hidden=320, group_size=2, mtp_heads=2, rms_eps=2e-8, tie_embeddings=False),
              page_size=16, gain_jitter=0.05, seed=14),
    # Matrices of the wide configurations are drawn with the standard deviation the sizes are specified with (0.02;
    # with 0.05 every product of 1536 inputs doubles the stream's scale and with it bfloat16's rounding error), and
    # their query projections are then multiplied by `sharpen`, so that attention weights are far from uniform and a
    # wrong key, mask or page moves the result.
    # the headline size's layer sizes (1536 wide, 12 query heads of 128 over 3, feed-forward 4096, two prediction
    # heads) with 2 of its 30 layers and a small vocabulary
    "E": dict(cfg=GqaMtpConfig(d_model=1536, vocab_size=1000, max_context=2304, rope_base=10000.0, n_heads=12,
                               n_layers=2, ffn_hidden=4096, group_size=4, mtp_heads=2, rms_eps=2e-8,
                               tie_embeddings=True),
              page_size=16, gain_jitter=0.1, seed=15, std=0.02, sharpen=2.0),
    # the attention geometries of the two larger sizes (16 heads of 128 over 4; 32 over 8) with one layer and a
    # narrow feed-forward
    "F": dict(cfg=GqaMtpConfig(d_model=2048, vocab_size=900, max_context=1536, rope_base=10000.0, n_heads=16,
                               n_layers=1, ffn_hidden=1408, group_size=4, mtp_heads=2, rms_eps=2e-8,
                               tie_embeddings=True),
              page_size=16, gain_jitter=0.1, seed=16, std=0.02, sharpen=2.0),
    "G": dict(cfg=GqaMtpConfig(d_model=4096, vocab_size=600, max_context=1024, rope_base=500000.0, n_heads=32,
                               n_layers=1, ffn_hidden=1024, group_size=4, mtp_heads=1, rms_eps=2e-8,
                               tie_embeddings=False),
              page_size=16, gain_jitter=0.1, seed=17, std=0.02, sharpen=2.0),
}

_folders: Dict[Tuple[str, str], str] = {}
_tmp = None


def model_folder(name: str, storage: str = "bfloat16") -> str:
    """A model folder of tiny configuration `name`, made once per test session in a temporary place."""
    global _tmp
    key = (name, storage)
    if key not in _folders:
        if _tmp is None:
            _tmp = tempfile.TemporaryDirectory(prefix="tis_amd_models_")
        t = TINY[name]
        _folders[key] = write_random_model(t["cfg"], t["seed"], os.path.join(_tmp.name, f"{name}_{storage}"),
                                           std=t.get("std", 0.05), gain_jitter=t["gain_jitter"], dtype=storage)
        if t.get("sharpen"):
            from safetensors.torch import load_file, save_file
            path = os.path.join(_folders[key], "model.safetensors")
            tensors = load_file(path)
            for n in tensors:
                if n.endswith("att.q_proj.weight"):
                    tensors[n] = (tensors[n].float() * t["sharpen"]).to(tensors[n].dtype)
            save_file(tensors, path)
    return _folders[key]


_plain_cache: Dict[Tuple[str, Tuple[int, ...]], Tuple[torch.Tensor, List[torch.Tensor]]] = {}


def plain_logits(folder: str, ids: Sequence[int]):
    """(main [T, V], [head i [T-1-i, V]]) from the plain implementation in float64, cached per sequence."""
    key = (folder, tuple(ids))
    if key not in _plain_cache:
        cfg, w = pm.read_model_folder(folder)
        _plain_cache[key] = pm.forward_all(list(ids), w, cfg)
    return _plain_cache[key]


def random_ids(vocab: int, n: int, seed: int) -> List[int]:
    rng = random.Random(seed)
    return [rng.randrange(vocab) for _ in range(n)]


# ---- traces: lists of steps in the replay program's format ------------------------------------------------

def whole_trace(reqs: Dict[str, List[int]]):
    """Each request alone and whole, one step each, every position wanted."""
    steps = []
    for i, (rid, ids) in enumerate(reqs.items()):
        steps.append({"step": i, "entries": [{"id": rid, "tokens": ids, "want": list(range(len(ids)))}], "end": [rid]})
    return steps


def tail_decode_trace(reqs: Dict[str, List[int]], tail: int = 32):
    """Most of each request in one step, then its last `tail` tokens one by one."""
    steps = []
    for rid, ids in reqs.items():
        head = max(1, len(ids) - tail)
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": ids[:head], "want": list(range(head))}],
                      "end": []})
        for p in range(head, len(ids)):
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": [ids[p]], "want": [0]}],
                          "end": [rid] if p == len(ids) - 1 else []})
        if head == len(ids):
            steps[-1]["end"] = [rid]
    return steps


def portions_trace(reqs: Dict[str, List[int]], seed: int = 0, sizes=(2, 3, 5, 7, 16, 17, 31, 2, 9)):
    """Each request alone, in portions of changing size, down to two tokens."""
    steps = []
    for rid, ids in reqs.items():
        p, k = 0, seed
        while p < len(ids):
            n = min(sizes[k % len(sizes)], len(ids) - p)
            k += 1
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": ids[p:p + n], "want": list(range(n))}],
                          "end": [rid] if p + n == len(ids) else []})
            p += n
    return steps


def mixed_trace(reqs: Dict[str, List[int]], max_live: int = 4, seed: int = 0, prompt_frac: float = 0.6):
    """Up to `max_live` requests at a time: portions of some beside single tokens of others, requests ending and
    new ones taking over their pages. Returns (steps, most tokens held at once rounded to 64 per request)."""
    rng = random.Random(seed)
    waiting = list(reqs.items())
    live: Dict[str, int] = {}            # id -> tokens fed
    steps = []
    peak = 0
    while waiting or live:
        while waiting and len(live) < max_live:
            rid, _ = waiting.pop(0)
            live[rid] = 0
        entries, ended = [], []
        for rid in list(live):
            ids = reqs[rid]
            fed = live[rid]
            if rng.random() < 0.15 and len(live) > 1:
                continue                                   # left out of this step, goes on later
            prompt_len = int(len(ids) * prompt_frac)
            if fed < prompt_len:
                n = min(rng.choice((2, 3, 5, 8, 13, 21)), prompt_len - fed)
            else:
                n = 1
            n = min(n, len(ids) - fed)
            entries.append({"id": rid, "tokens": ids[fed:fed + n], "want": list(range(n))})
            live[rid] = fed + n
            if live[rid] == len(ids):
                ended.append(rid)
        peak = max(peak, sum(-(-max(v, 1) // 64) * 64 for v in live.values()))
        if entries:
            steps.append({"step": len(steps), "entries": entries, "end": ended})
        for rid in ended:
            del live[rid]
    return steps, peak


def wanted_keys(steps, n_heads: int):
    """What a trace asks for: the (id, position) of every wanted place, and for every prediction head the
    (id, head, head position) it owes there: head i answers a wanted position p with its row p - 1 - i, once
    that is a position at all."""
    fed: Dict[str, int] = {}
    main, heads = set(), set()
    for st in steps:
        for e in st["entries"]:
            start = fed.get(e["id"], 0)
            for i in e["want"]:
                main.add((e["id"], start + i))
                for hi in range(n_heads):
                    if start + i - 1 - hi >= 0:
                        heads.add((e["id"], hi, start + i - 1 - hi))
            fed[e["id"]] = start + len(e["tokens"])
        for rid in st["end"]:
            fed.pop(rid, None)
    return main, heads


def run_trace(engine, steps, heads: bool = True):
    """Drive the engine's step function; returns {(id, position): logits} and {(id, head, head position): logits}."""
    main: Dict[Tuple[str, int], torch.Tensor] = {}
    head_out: Dict[Tuple[str, int, int], torch.Tensor] = {}
    for st in steps:
        entries = [(e["id"], e["tokens"], e["want"]) for e in st["entries"]]
        starts = {e["id"]: (engine.fed(e["id"]) if e["id"] in engine.requests else 0) for e in st["entries"]}
        res = engine.step(entries, heads=heads)
        lg = res.logits.cpu()
        hl = [h.cpu() for h in res.head_logits] if res.head_logits else []
        row = 0
        for e in st["entries"]:
            for i in e["want"]:
                pos = starts[e["id"]] + i
                main[(e["id"], pos)] = lg[row]
                for hi, h in enumerate(hl):
                    if res.head_valid[hi][row]:
                        head_out[(e["id"], hi, pos - 1 - hi)] = h[row]
                row += 1
        for rid in st["end"]:
            engine.close(rid)
    return main, head_out


def compare_with_plain(folder, reqs, main, head_out, tol, n_heads, steps=None):
    """Largest absolute difference against the plain implementation, asserted below `tol`, with the place named.
    With `steps` (the trace that was run) also: everything the trace asked for came back, and nothing else."""
    if steps is not None:
        want_main, want_heads = wanted_keys(steps, n_heads)
        assert set(main) == want_main, f"main logits: missing {sorted(want_main - set(main))[:5]}, " \
                                       f"unasked {sorted(set(main) - want_main)[:5]}"
        assert set(head_out) == want_heads, f"head logits: missing {sorted(want_heads - set(head_out))[:5]}, " \
                                            f"unasked {sorted(set(head_out) - want_heads)[:5]}"
        for rid, hi, p in want_heads:
            assert p < len(reqs[rid]) - 1 - hi
    worst = (0.0, None)
    for rid, ids in reqs.items():
        pm_main, pm_heads = plain_logits(folder, ids)
        for p in range(len(ids)):
            if (rid, p) in main:
                d = (main[(rid, p)].double() - pm_main[p]).abs().max().item()
                if not d <= worst[0]:
                    worst = (d, ("main", rid, p))
        for hi in range(n_heads):
            for p in range(pm_heads[hi].shape[0]):
                if (rid, hi, p) in head_out:
                    d = (head_out[(rid, hi, p)].double() - pm_heads[hi][p]).abs().max().item()
                    if not d <= worst[0]:
                        worst = (d, (f"head{hi}", rid, p))
    assert worst[0] <= tol, f"largest difference {worst[0]:.3e} at {worst[1]} exceeds {tol:.1e}"
    return worst


def first_wrong(folder, reqs, main, tol):
    """The first (request, position) whose main logits differ by more than tol: where to look when a schedule fails."""
    for rid, ids in reqs.items():
        pm_main, _ = plain_logits(folder, ids)
        for p in range(len(ids)):
            if (rid, p) in main and not (main[(rid, p)].double() - pm_main[p]).abs().max().item() <= tol:
                return rid, p
    return None


SLOT_CASES = [(1, "final", None), (2, "final", None), (2, "cur", 80), (3, "cur", 96)]   # max_batch, plan, pool tokens


def slot_pressure_workload(name: str):
    """Five greedy requests of different prompt and output lengths, so that in a batch the newest often finishes first
    and its successor takes its slot: (folder, prompts, sampling params, the plain model's tokens)."""
    from tiny_inference_server_amd.sampling import SamplingParams
    folder = model_folder(name, "float32")
    cfg, w = pm.read_model_folder(folder)
    lens, new = [30, 7, 12, 19, 5], [24, 5, 9, 14, 20]
    prompts = [random_ids(cfg["vocab"], n, 190 + i) for i, n in enumerate(lens)]
    params = [SamplingParams(max_new_tokens=k, temperature=0.0, ignore_eos=True) for k in new]
    want = [pm.greedy_generate(p, k, w, cfg) for p, k in zip(prompts, new)]
    return folder, prompts, params, want


# ---- many sampled requests through the scheduler: more live requests than captured steps have exact shapes for ------

def sampled_workload(name: str, n_req: int, seed: int, temperature: float = 0.3, rep_penalty: float = 1.3):
    """`n_req` requests of mixed prompt and output lengths, sampled with a temperature and a repetition penalty, each
    from its own random stream: (prompts, sampling params)."""
    from tiny_inference_server_amd.sampling import SamplingParams
    rng = random.Random(seed)
    vocab = TINY[name]["cfg"].vocab_size
    prompts = [random_ids(vocab, rng.randint(18, 60), seed + 1 + i) for i in range(n_req)]
    params = [SamplingParams(max_new_tokens=rng.randint(10, 22), temperature=temperature, rep_penalty=rep_penalty,
                             seed=seed + i, ignore_eos=True) for i in range(n_req)]
    return prompts, params


def fill_cache_with_nan(engine) -> None:
    """Whatever a kernel reads of a page that its row may not see is then not a number."""
    for g in engine.cache.groups.values():
        g.storage.fill_(float("nan"))


def watch_decode_steps(engine):
    """Records, for every step of single tokens that goes through the captured-step path, (requests in the step,
    whether it was replayed from a kept step). Returns the list that fills up."""
    seen = []
    inner = engine._decode_step

    def watching(batch_entries):
        before = engine.graph_replays
        out = inner(batch_entries)
        seen.append((len(batch_entries), engine.graph_replays > before))
        return out
    engine._decode_step = watching
    return seen


def check_sampled_tokens(folder, prompts, params, outs, slack: float):
    """Every generated token against the reference's sampling rule (server.py:22-50) on the plain model's logits for
    the tokens before it, with the request's own uniform number u. The draw inverts the cumulative distribution in
    token order and is monotone in u, so a token must lie between the plain draws at u - slack and u + slack: `slack`
    is what the compute dtype's rounding may move the cumulative mass by (1e-5 in 32-bit). Returns (tokens checked,
    tokens equal to the plain draw at u itself)."""
    from tiny_inference_server_amd.sampling import uniform_for
    cfg, w = pm.read_model_folder(folder)
    checked = equal = 0
    for prompt, sp, out in zip(prompts, params, outs):
        assert len(out) == sp.max_new_tokens
        ids = list(prompt) + list(out)
        logits = pm.logits_of(pm.trunk_hidden(ids[:-1], w, cfg), w, cfg)
        for i, tok in enumerate(out):
            p = len(prompt) - 1 + i
            probs = pm.sampling_probs(logits[p], sp.temperature, sp.top_k, sp.top_p, sp.rep_penalty, ids[:p + 1])
            u = uniform_for(sp.seed, i)
            lo = pm.pick_by_uniform(probs, max(0.0, u - slack))
            hi = pm.pick_by_uniform(probs, u + slack) if u + slack < 1.0 else int(torch.nonzero(probs)[-1])
            assert lo <= tok <= hi, (prompt[:3], i, tok, lo, hi)
            assert probs[tok] > 0
            checked += 1
            equal += tok == pm.pick_by_uniform(probs, u)
    return checked, equal

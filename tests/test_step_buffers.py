"""Steps kept in fixed buffers (the host side of captured graphs), run on the CPU stand-in for the kernels.

A captured decode step keeps its integer arrays in one buffer; while the same requests come again in the same order
only tokens, positions, write slots and newly taken pages are rewritten. "The same requests" must mean the requests
themselves: a cache slot is handed to request after request, and a successor that holds no more pages than its
predecessor did would otherwise run on the predecessor's block table (the policy being followed: finished requests
leave, queued ones take their places, reference server.py:286-292).
"""
import pytest
import torch

import helpers as H
from tiny_inference_server_amd.engine import Engine
from torch_ops import TorchOps

TOL = {"float32": 2e-5, "bfloat16": 2e-2}


def engine_for(name, dtype, max_tokens, max_requests, graphs=True):
    folder = H.model_folder(name, "float32" if dtype == "float32" else "bfloat16")
    ops = TorchOps(dtype=torch.float32 if dtype == "float32" else torch.bfloat16, graphs=graphs)
    return folder, Engine(folder, dtype=dtype, page_size=H.TINY[name]["page_size"], max_tokens=max_tokens,
                          max_requests=max_requests, ops=ops)


def scale_of(folder, reqs):
    return max(1.0, max(H.plain_logits(folder, ids)[0].abs().max().item() for ids in reqs.values()))


def one_after_the_other(reqs, prompt):
    """Every request alone: `prompt` tokens in one step, the rest one by one; the next request starts when it ends."""
    steps = []
    for rid, ids in reqs.items():
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": ids[:prompt], "want": [prompt - 1]}], "end": []})
        for p in range(prompt, len(ids)):
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": [ids[p]], "want": [0]}],
                          "end": [rid] if p == len(ids) - 1 else []})
    return steps


@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("B", "float32"), ("D", "bfloat16")])
def test_a_slot_that_changes_hands_gets_its_new_owners_pages(name, dtype):
    """One slot only, so every request follows its predecessor into it; the second is shorter than the first and the
    third longer, and all decode through the same captured shape."""
    vocab = H.TINY[name]["cfg"].vocab_size
    reqs = {f"s{i}": H.random_ids(vocab, n, 90 + i) for i, n in enumerate([70, 40, 75, 41])}
    folder, eng = engine_for(name, dtype, max_tokens=256, max_requests=1)
    assert eng.use_graphs
    steps = one_after_the_other(reqs, 9)
    main, _ = H.run_trace(eng, steps, heads=False)
    assert eng.graph_replays > 100
    assert set(main) == {(rid, p) for rid, ids in reqs.items() for p in range(8, len(ids))}
    H.compare_with_plain(folder, reqs, main, {}, TOL[dtype] * scale_of(folder, reqs), 0, steps)
    eng.cache.check()
    assert eng.free_pages() == eng.total_pages()


def test_quick_update_is_refused_after_a_slot_changed_hands():
    """The buffer of a captured step answers for the requests it was filled with, not for their slots."""
    name = "A"
    vocab = H.TINY[name]["cfg"].vocab_size
    folder, eng = engine_for(name, "float32", max_tokens=256, max_requests=1)
    a, b = H.random_ids(vocab, 70, 1), H.random_ids(vocab, 30, 2)
    eng.step([("a", a[:60], [])])
    for p in range(60, 64):
        eng.step([("a", [a[p]], [0])])
    graph = next(iter(eng._graphs.values()))
    slot_a = eng.requests["a"][0]
    held = graph.occupants
    assert graph.holds(held)
    eng.close("a")
    eng.step([("b", b[:20], [])])
    assert eng.requests["b"][0] == slot_a               # the same slot ...
    assert not graph.holds(eng._occupants([type("E", (), {"slot": slot_a})()]))   # ... but not the same request
    replays = eng.graph_replays
    out = eng.step([("b", [b[20]], [0])])
    assert eng.graph_replays == replays + 1             # refilled in full and replayed
    want = H.plain_logits(folder, b)[0][20]
    assert (out.logits[0].double() - want).abs().max().item() <= 2e-5 * max(1.0, want.abs().max().item())
    # the buffer's block-table line is b's now
    (t_off, (rows, width)), = [graph.table_at[g] for g in graph.table_at][:1]
    line = graph.host.numpy()[t_off:t_off + width]
    table = next(iter(eng.cache.groups.values())).tables[slot_a]
    assert list(line[:len(table)]) == table


@pytest.mark.parametrize("name,dtype", [("B", "float32"), ("D", "bfloat16")])
@pytest.mark.parametrize("seed", [21, 22])
def test_mixed_schedules_through_step_buffers(name, dtype, seed):
    """Random mixed schedules with exactly as many slots as live requests: requests end, others take their slots and
    pages, and decode steps of the same shape keep coming."""
    import random
    rng = random.Random(seed)
    vocab = H.TINY[name]["cfg"].vocab_size
    lengths = [rng.choice((3, 17, 33, 40, 64, 65, 80)) for _ in range(7)]
    reqs = {f"r{i}": H.random_ids(vocab, n, seed * 100 + i) for i, n in enumerate(lengths)}
    live = rng.randint(1, 3)
    steps, peak = H.mixed_trace(reqs, max_live=live, seed=seed, prompt_frac=0.3)
    folder, eng = engine_for(name, dtype, max_tokens=peak, max_requests=live)
    main, _ = H.run_trace(eng, steps, heads=False)
    assert eng.graph_replays > 0
    H.compare_with_plain(folder, reqs, main, {}, TOL[dtype] * scale_of(folder, reqs), 0, steps)
    eng.cache.check()
    assert eng.free_pages() == eng.total_pages()


@pytest.mark.parametrize("name", ["A", "B"])
@pytest.mark.parametrize("max_batch,plan,pool", H.SLOT_CASES)
def test_generation_with_as_many_slots_as_requests(name, max_batch, plan, pool):
    """The scheduler above an engine that has exactly max_batch slots: finished and preempted requests hand their
    slots on, decode steps of the same shape keep coming, and the greedy tokens are the plain model's."""
    from tiny_inference_server_amd.engine.generate import generate
    folder, prompts, params, want = H.slot_pressure_workload(name)
    ps = H.TINY[name]["page_size"]
    longest = max(len(p) + sp.max_new_tokens for p, sp in zip(prompts, params))
    eng = Engine(folder, dtype="float32", page_size=ps, max_requests=max_batch, ops=TorchOps(graphs=True),
                 max_tokens=pool if pool is not None else max_batch * (-(-longest // ps) * ps), run_heads=False)
    got, s = generate(eng, prompts, params=params, max_batch=max_batch, token_budget=16, plan=plan, return_scheduler=True)
    assert eng.graph_replays > 0
    assert (s.preempts > 0) == (pool is not None)
    assert got == want
    eng.cache.check()
    assert eng.free_pages() == eng.total_pages()


class PlanningOps(TorchOps):
    """The stand-in with the attention mixer's host planning switched on, as the real operations have it: the plan's
    arrays travel with the step, the stand-in's attention ignores them."""

    def plan_attention_mode(self, seq_rows, window=0):
        from tiny_inference_server_amd.ops.hip_ops import uneven_lengths
        return "uneven" if uneven_lengths(seq_rows) else None

    def plan_attention(self, n_heads, n_kv_heads, head_dim, seq_rows, add, mode=None, window=0):
        from tiny_inference_server_amd.ops.hip_ops import decode_items
        if mode != "uneven":
            return {}
        entries, most = decode_items(seq_rows, n_heads, n_kv_heads, head_dim)
        return {("attention_decode_items", n_heads, n_kv_heads): (add(entries), len(entries), most)}


def test_parts_plan_again_for_every_replay_of_a_captured_step():
    """A captured step of requests that differ widely in length carries a work list planned on the host. When the
    same requests come again the list is planned again, for the new positions, into its place in the step's buffer:
    what every step ran on (the device's copy of the buffer) is, integer for integer, what a fresh plan of that step
    holds. (The host's copy is by then already filled for the step after, ahead of time: all but its tokens.)"""
    from tiny_inference_server_amd.engine.batch import Entry, first_stage_rows, plan_step_batch
    name = "D"
    folder = H.model_folder(name, "float32")
    cfg = H.TINY[name]["cfg"]
    lengths = [500, 30, 90, 41]
    reqs = {f"p{i}": H.random_ids(cfg.vocab_size, n, 140 + i) for i, n in enumerate(lengths)}
    eng = Engine(folder, dtype="float32", page_size=16, max_tokens=1024, max_requests=4, ops=PlanningOps(graphs=True))
    for rid, ids in reqs.items():
        eng.step([(rid, ids[:-24], [])])
    main, checked, ahead = {}, 0, 0
    for t in range(24):
        entries = [(rid, [ids[len(ids) - 24 + t]], [0]) for rid, ids in reqs.items()]
        slots = [(eng.requests[rid][0], eng.requests[rid][1]) for rid in reqs]
        out = eng.step(entries)
        for k, rid in enumerate(reqs):
            main[(rid, len(reqs[rid]) - 24 + t)] = out.logits[k].float().clone()
        graphs = [g for key, g in eng._graphs.items() if key[0] != "step" and key[2] is not None]
        if not graphs:
            continue                                        # the shape's first step runs as it is
        graph = graphs[0]
        batch_entries = [Entry(s, fed, [e[1][0]], [0]) for (s, fed), e in zip(slots, entries)]
        mode = eng.model.plan_mode(first_stage_rows(batch_entries))
        assert mode is not None and mode == graph.mode
        width = graph.table_at[next(iter(graph.table_at))][1][1]
        fresh = plan_step_batch(batch_entries, eng.model.lags, eng.model.reads_previous, eng.cache,
                                eng.spec.max_context, eng.model.plan_rows, table_width=width, mode=mode)
        assert fresh.layout() == graph.layout
        want = torch.zeros_like(graph.host)
        fresh.packer.fill(want)
        assert torch.equal(graph.dev[:fresh.packer.total].cpu(), want[:fresh.packer.total]), t
        if graph._ahead is not None:            # (not after the step that made the graph)
            assert graph._ahead[0].tolist() == [fed + 1 for _, fed in slots]
            ahead += 1
        checked += 1
    assert checked >= 20 and eng.graph_replays >= 20 and ahead >= 18
    H.compare_with_plain(folder, reqs, main, {}, TOL["float32"] * scale_of(folder, reqs), 0)


def shrinking_batch(reqs, prompt):
    """All requests decode side by side after their prompts; they are of different lengths, so the batch shrinks one
    request at a time."""
    steps = [{"step": i, "entries": [{"id": rid, "tokens": ids[:prompt], "want": []}], "end": []}
             for i, (rid, ids) in enumerate(reqs.items())]
    fed = {rid: prompt for rid in reqs}
    while any(fed[r] < len(reqs[r]) for r in reqs):
        live = [r for r in reqs if fed[r] < len(reqs[r])]
        steps.append({"step": len(steps), "entries": [{"id": r, "tokens": [reqs[r][fed[r]]], "want": [0]} for r in live],
                      "end": [r for r in live if fed[r] + 1 == len(reqs[r])]})
        for r in live:
            fed[r] += 1
    return steps


@pytest.mark.parametrize("backend", [pytest.param("hip", marks=pytest.mark.gpu), "torch"])
@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("B", "float32"), ("D", "bfloat16")])
def test_a_batch_that_shrinks_request_by_request_meets_few_shapes(name, dtype, backend):
    """Thirteen requests decode side by side and end one after the other. Steps of nine and more are filled up to 16
    lines with the cache manager's own request, so sizes 13 down to 9 share one captured shape (two with the table
    width growing), sizes 8 down to 1 have their own; the filler's lines never come back, and every request's logits
    equal the plain model's, also right after a neighbour has left."""
    vocab = H.TINY[name]["cfg"].vocab_size
    reqs = {f"k{i}": H.random_ids(vocab, 24 + 3 * i, 700 + i) for i in range(13)}
    page = H.TINY[name]["page_size"]
    peak = sum(-(-len(ids) // page) * page for ids in reqs.values())
    if backend == "torch":
        folder, eng = engine_for(name, dtype, max_tokens=peak, max_requests=13)
    else:
        folder = H.model_folder(name, "float32" if dtype == "float32" else "bfloat16")
        eng = Engine(folder, dtype=dtype, page_size=page, max_tokens=peak, max_requests=13)
    assert eng.use_decode_graphs and eng.cache.spare_slot == 13
    steps = shrinking_batch(reqs, 20)
    main, _ = H.run_trace(eng, steps, heads=False)
    H.compare_with_plain(folder, reqs, main, {}, TOL[dtype] * scale_of(folder, reqs), 0, steps)
    sizes = sorted({k[0] for k in eng._graphs if k[0] != "step"} | {k[0] for k in eng._graph_seen if k[0] != "step"})
    assert sizes == [1, 2, 3, 4, 5, 6, 7, 8, 16]
    assert eng.graph_replays > 30
    eng.cache.check()
    assert eng.free_pages() == eng.total_pages() and eng.cache.n_live == 0

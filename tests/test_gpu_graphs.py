"""Captured decode steps against the same steps run kernel by kernel, replay after replay."""
import pytest
import torch

import helpers as H
from tiny_inference_server_amd.engine import Engine

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("name", ["C", "D", "A"])
def test_graph_replays_match_eager_steps(name):
    """Several requests decode together; each replay is checked against an engine without graphs and against the
    plain implementation, with eager prompt work and synchronisations between the replays."""
    folder = H.model_folder(name, "bfloat16")
    vocab = H.TINY[name]["cfg"].vocab_size
    reqs = {f"r{i}": H.random_ids(vocab, n, 40 + i) for i, n in enumerate([60, 47, 75])}
    prompt = 20
    engines = {flag: Engine(folder, dtype="bfloat16", page_size=H.TINY[name]["page_size"], max_tokens=512,
                            max_requests=8, use_graphs=flag) for flag in (True, False)}
    got = {True: {}, False: {}}
    for flag, eng in engines.items():
        for rid, ids in reqs.items():
            eng.step([(rid, ids[:prompt], [])])
        for p in range(prompt, 47):
            live = [rid for rid, ids in reqs.items() if p < len(ids)]
            out = eng.step([(rid, [reqs[rid][p]], [0]) for rid in live])
            lg = out.logits.float().cpu().clone()
            for k, rid in enumerate(live):
                got[flag][(rid, p)] = lg[k]
            if p % 5 == 0:
                # eager work of another shape between replays: a new request's prompt, then its end
                eng.step([("extra", reqs["r0"][:9], [8])])
                eng.close("extra")
                torch.cuda.synchronize()
    assert engines[True].graph_replays >= 20 and engines[False].graph_replays == 0
    tol = 2e-2 * max(1.0, max(H.plain_logits(folder, ids)[0].abs().max().item() for ids in reqs.values()))
    assert set(got[True]) == set(got[False]) == {(r, p) for r, ids in reqs.items() for p in range(prompt, min(47, len(ids)))}
    H.compare_with_plain(folder, reqs, got[True], {}, tol, 0)
    H.compare_with_plain(folder, reqs, got[False], {}, tol, 0)
    # two bfloat16 runs that are each within tol of the plain result are within 2 tol of each other; the graph
    # cuts the keys into other splits than the eager step, so they are not bit-equal
    for key in got[False]:
        assert (got[True][key] - got[False][key]).abs().max().item() <= 2 * tol, key


@pytest.mark.parametrize("max_graphs", [32, 2])
def test_graph_survives_changing_batches(max_graphs):
    """Requests join and leave: graphs of several shapes are captured and reused; results stay right, also when
    only two graphs may be kept and the least recently used one goes each time a third shape comes."""
    name = "D"
    folder = H.model_folder(name, "bfloat16")
    vocab = H.TINY[name]["cfg"].vocab_size
    reqs = {f"q{i}": H.random_ids(vocab, n, 60 + i) for i, n in enumerate([50, 30, 44, 38])}
    eng = Engine(folder, dtype="bfloat16", page_size=16, max_tokens=512, max_requests=8)
    eng.max_graphs = eng.max_decode_graphs = max_graphs
    main = {}
    for rid, ids in reqs.items():
        eng.step([(rid, ids[:10], [])])
    fed = {rid: 10 for rid in reqs}
    while any(fed[r] < len(reqs[r]) for r in reqs):
        live = [r for r in reqs if fed[r] < len(reqs[r])]
        out = eng.step([(r, [reqs[r][fed[r]]], [0]) for r in live])
        lg = out.logits.float().cpu().clone()
        for k, r in enumerate(live):
            main[(r, fed[r])] = lg[k]
            fed[r] += 1
    assert set(main) == {(r, p) for r, ids in reqs.items() for p in range(10, len(ids))}
    decode_graphs = [k for k in eng._graphs if k[0] != "step"]          # (the prompts' portions may have one of their own)
    assert min(3, max_graphs) <= len(decode_graphs) <= max_graphs and eng.graph_replays >= 30
    H.compare_with_plain(folder, reqs, main, {}, 2e-2 * max(1.0, max(
        H.plain_logits(folder, ids)[0].abs().max().item() for ids in reqs.values())), 0)


@pytest.mark.parametrize("name", ["B", "D"])
def test_repeated_prompt_steps_are_replayed(name):
    """A step of the same shape (two prompts of fixed lengths in one batch, the same places wanted) comes again and
    again with other tokens, in other slots and pages, with eager steps of other shapes in between: from its third
    occurrence it is replayed from a graph, and every occurrence must match the plain implementation."""
    folder = H.model_folder(name, "bfloat16")
    vocab = H.TINY[name]["cfg"].vocab_size
    eng = Engine(folder, dtype="bfloat16", page_size=H.TINY[name]["page_size"], max_tokens=512, max_requests=8)
    lengths = (41, 30)
    worst_scale = 1.0
    for rep in range(7):
        reqs = {f"p{rep}_{i}": H.random_ids(vocab, n, 300 + 10 * rep + i) for i, n in enumerate(lengths)}
        if rep % 2:
            # something else lives in the cache meanwhile, so slots and pages differ from the captured step's
            eng.step([("other", H.random_ids(vocab, 13 + rep, 77), [0])])
        out = eng.step([(rid, ids, [0, len(ids) // 2, len(ids) - 1]) for rid, ids in reqs.items()])
        lg = out.logits.float().cpu().clone()
        torch.cuda.synchronize()
        main = {}
        for k, (rid, ids) in enumerate(reqs.items()):
            for j, p in enumerate((0, len(ids) // 2, len(ids) - 1)):
                main[(rid, p)] = lg[3 * k + j]
        scale = max(1.0, max(H.plain_logits(folder, ids)[0].abs().max().item() for ids in reqs.values()))
        H.compare_with_plain(folder, reqs, main, {}, 2e-2 * scale, 0)
        for rid in reqs:
            eng.close(rid)
        if rep % 2:
            eng.close("other")
    assert eng.graph_replays >= 4
    eng.cache.check()
    assert eng.free_pages() == eng.total_pages()


def test_tiles_beside_items_on_two_streams_eager_and_replayed():
    """A step of one long portion (tiles of a workgroup, on the library's second stream) beside a shorter one and three
    decoded tokens (items, one wave each, on the first): the two kernels run side by side and meet again before the
    merge. The same shape comes four times with other tokens; the first runs kernel by kernel, the last from a captured
    graph whose branches fork and join. Logits at the ends of both portions and of the decoded tokens equal the plain
    model's every time they are checked."""
    from tiny_inference_server_amd.ops import hip_ops
    name = "E"                                            # the headline model's layer sizes: 12 heads of 128 over 3
    folder = H.model_folder(name, "bfloat16")
    cfg = H.TINY[name]["cfg"]
    eng = Engine(folder, dtype="bfloat16", page_size=16, max_tokens=4096, max_requests=8)
    long, short, deep = 1700, 300, 70
    seen = []
    plan_attention = eng.ops.plan_attention

    def spy(*a, **k):
        out = plan_attention(*a, **k)
        seen.extend((v[1], v[3]) for key, v in out.items() if key[0] == "attention_items")
        return out
    eng.ops.plan_attention = spy
    for rep in range(4):
        reqs = {f"t{rep}_{i}": H.random_ids(cfg.vocab_size, n, 500 + 10 * rep + i) for i, n in enumerate([long, short, deep, deep + 3, deep + 9])}
        names = list(reqs)
        for rid in names[2:]:                             # three requests already deep enough to decode
            eng.step([(rid, reqs[rid][:-1], [])])
        seen.clear()
        out = eng.step([(names[0], reqs[names[0]], [long - 1]), (names[1], reqs[names[1]], [0, short - 1])] +
                       [(rid, reqs[rid][-1:], [0]) for rid in names[2:]])
        assert any(items > 0 and tiles > 0 for items, tiles in seen)          # both kernels had work in this step
        lg = out.logits.float().cpu().clone()
        torch.cuda.synchronize()
        if rep in (0, 3):
            main = {(names[0], long - 1): lg[0], (names[1], 0): lg[1], (names[1], short - 1): lg[2]}
            main.update({(rid, len(reqs[rid]) - 1): lg[3 + k] for k, rid in enumerate(names[2:])})
            scale = max(1.0, max(H.plain_logits(folder, ids)[0].abs().max().item() for ids in reqs.values()))
            H.compare_with_plain(folder, reqs, main, {}, 2e-2 * scale, 0)
        for rid in names:
            eng.close(rid)
    assert eng.graph_replays >= 1 and hip_ops._side_streams
    eng.cache.check()
    assert eng.free_pages() == eng.total_pages()


@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("B", "float32"), ("D", "bfloat16"), ("C", "bfloat16")])
def test_requests_follow_each_other_through_one_slot(name, dtype):
    """As many slots as live requests: one. Every request takes over its predecessor's slot at the same place in the
    batch; the second holds fewer pages than the first did, the third more. A captured step must run on the new
    owner's block table (finished requests leave and queued ones take their places: reference server.py:286-292)."""
    from test_step_buffers import one_after_the_other
    folder = H.model_folder(name, "float32" if dtype == "float32" else "bfloat16")
    vocab = H.TINY[name]["cfg"].vocab_size
    reqs = {f"s{i}": H.random_ids(vocab, n, 90 + i) for i, n in enumerate([70, 40, 75, 41])}
    eng = Engine(folder, dtype=dtype, page_size=H.TINY[name]["page_size"], max_tokens=256, max_requests=1)
    assert eng.use_graphs
    steps = one_after_the_other(reqs, 9)
    main, _ = H.run_trace(eng, steps, heads=False)
    assert eng.graph_replays > 100
    tol = (2e-5 if dtype == "float32" else 2e-2) * max(1.0, max(
        H.plain_logits(folder, ids)[0].abs().max().item() for ids in reqs.values()))
    H.compare_with_plain(folder, reqs, main, {}, tol, 0, steps)
    eng.cache.check()
    assert eng.free_pages() == eng.total_pages()


@pytest.mark.parametrize("name", ["A", "B"])
@pytest.mark.parametrize("max_batch,plan,pool", H.SLOT_CASES)
def test_generation_with_as_many_slots_as_requests(name, max_batch, plan, pool):
    """generate() gives the engine exactly max_batch slots. Requests of different lengths, the newest of a batch
    finishing first, its successor taking its slot; with plan "cur" on a small pool requests are preempted and
    admitted again into slots others have used meanwhile. Greedy tokens in 32-bit equal the plain model's."""
    from tiny_inference_server_amd.engine.generate import generate
    folder, prompts, params, want = H.slot_pressure_workload(name)
    got, s = generate(folder, prompts, params=params, dtype="float32", tokens_per_block=H.TINY[name]["page_size"],
                      max_batch=max_batch, token_budget=16, plan=plan, pool_tokens=pool, return_scheduler=True)
    assert s.engine.cache.max_requests == max_batch
    assert s.engine.graph_replays > 0
    assert (s.preempts > 0) == (pool is not None)
    assert got == want
    s.engine.cache.check()
    assert s.engine.free_pages() == s.engine.total_pages()


@pytest.mark.parametrize("name", ["E", "D"])
def test_decoding_requests_of_very_different_lengths_from_captured_graphs(name):
    """Eighteen requests of 30 to 2,000 tokens decode side by side: their key splits are planned request by request on
    the host (the longest would otherwise run on alone), the plan is made again for every replay of the captured step,
    and a request that leaves changes the batch's shape; once fewer than sixteen are left all get the same splits. Logits equal the plain model's at every decoded position; the same
    trace without graphs gives the same plan and, within rounding, the same logits."""
    from tiny_inference_server_amd.ops import hip_ops
    folder = H.model_folder(name, "bfloat16")
    cfg = H.TINY[name]["cfg"]
    lengths = [2000, 30, 420, 64, 1100, 47] if cfg.max_context >= 2304 else [600, 30, 120, 64, 350, 47]
    tail = [24, 10, 24, 24, 16, 24]                       # tokens decoded one by one at the end of each request
    lengths, tail = lengths + [90 + 11 * i for i in range(12)], tail + [24 - i % 3 for i in range(12)]
    reqs = {f"u{i}": H.random_ids(cfg.vocab_size, n, 130 + i) for i, n in enumerate(lengths)}
    peak = sum(-(-n // 16) * 16 for n in lengths)
    got = {}
    for graphs in (True, False):
        eng = Engine(folder, dtype="bfloat16", page_size=16, max_tokens=peak, max_requests=len(reqs), use_graphs=graphs)
        main = {}
        for (rid, ids), t in zip(reqs.items(), tail):
            for p in range(0, len(ids) - t, 512):
                eng.step([(rid, ids[p:min(p + 512, len(ids) - t)], [])])
        fed = {rid: len(ids) - t for (rid, ids), t in zip(reqs.items(), tail)}
        planned = 0
        while any(fed[r] < len(reqs[r]) for r in reqs):
            live = [r for r in reqs if fed[r] < len(reqs[r])]
            rows = [(k, fed[r], 1) for k, r in enumerate(live)]
            planned += hip_ops.uneven_lengths(rows) and hip_ops.planned_list_pays(len(live), cfg.n_kv_heads)
            out = eng.step([(r, [reqs[r][fed[r]]], [0]) for r in live])
            lg = out.logits.float().cpu().clone()
            for k, r in enumerate(live):
                main[(r, fed[r])] = lg[k]
                fed[r] += 1
        assert planned >= 20                               # most of these steps take the planned lists
        if graphs:
            assert eng.graph_replays >= 15 and any(k[0] != "step" and k[2] is not None for k in eng._graphs)
        got[graphs] = main
        tol = 2e-2 * max(1.0, max(H.plain_logits(folder, ids)[0].abs().max().item() for ids in reqs.values()))
        H.compare_with_plain(folder, reqs, main, {}, tol, 0)
        assert set(main) == {(r, p) for (r, ids), t in zip(reqs.items(), tail) for p in range(len(ids) - t, len(ids))}
    for key in got[True]:
        assert (got[True][key] - got[False][key]).abs().max().item() <= 2 * tol, key

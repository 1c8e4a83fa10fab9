"""The engine against the plain implementation under every way of cutting and batching the same requests.

The same tests run twice: on the GPU with the HIP kernels (marked gpu), in 32-bit and in bfloat16, and on
the CPU with the plain torch stand-ins for the kernels (tests/torch_ops.py), which checks the step function,
the batch builder and the cache without a GPU. Tolerances are fixed: 2e-5 of the logits' scale in 32-bit,
2e-2 in bfloat16 (bfloat16 keeps 8 bits; the measured error of a correct run is about a fifth of that).
"""
import pytest
import torch

import helpers as H
from tiny_inference_server_amd.engine import Engine

TOL = {"float32": 2e-5, "bfloat16": 2e-2}


def backends():
    return [pytest.param("hip", marks=pytest.mark.gpu), pytest.param("torch", marks=[])]


def make_engine(name, dtype, backend, max_tokens, max_requests=4):
    folder = H.model_folder(name, "float32" if dtype == "float32" else "bfloat16")
    ops = None
    if backend == "torch":
        from torch_ops import TorchOps
        ops = TorchOps(dtype=torch.float32 if dtype == "float32" else torch.bfloat16)
    eng = Engine(folder, dtype=dtype, page_size=H.TINY[name]["page_size"], max_tokens=max_tokens,
                 max_requests=max_requests, ops=ops)
    return folder, eng


def requests_for(name, lengths, seed):
    vocab = H.TINY[name]["cfg"].vocab_size
    return {f"r{i}": H.random_ids(vocab, n, seed * 100 + i) for i, n in enumerate(lengths)}


def scale_of(folder, reqs):
    return max(1.0, max(H.plain_logits(folder, ids)[0].abs().max().item() for ids in reqs.values()))


CASES = [("A", "float32"), ("B", "float32"), ("A", "bfloat16"), ("B", "bfloat16"), ("C", "bfloat16"),
         ("D", "bfloat16"), ("D", "float32")]
# the layer sizes of the headline model and the attention geometries of the two larger ones: on the GPU only (their
# plain results alone take the CPU a while)
BIG_CASES = [pytest.param(n, "bfloat16", "hip", marks=pytest.mark.gpu) for n in ("E", "F", "G")]


@pytest.mark.parametrize("backend", backends())
@pytest.mark.parametrize("name,dtype", CASES)
def test_whole_requests(name, dtype, backend):
    reqs = requests_for(name, [5, 17, 33, 1, 2, 70], seed=1)
    folder, eng = make_engine(name, dtype, backend, max_tokens=128)
    steps = H.whole_trace(reqs)
    main, heads = H.run_trace(eng, steps)
    H.compare_with_plain(folder, reqs, main, heads, TOL[dtype] * scale_of(folder, reqs), eng.config.mtp_heads, steps)
    eng.cache.check()
    assert eng.free_pages() == eng.total_pages()


@pytest.mark.parametrize("backend", backends())
@pytest.mark.parametrize("name,dtype", CASES)
def test_prefill_then_decode_one_by_one(name, dtype, backend):
    reqs = requests_for(name, [75, 40, 33], seed=2)
    folder, eng = make_engine(name, dtype, backend, max_tokens=128)
    steps = H.tail_decode_trace(reqs, tail=32)
    main, heads = H.run_trace(eng, steps)
    H.compare_with_plain(folder, reqs, main, heads, TOL[dtype] * scale_of(folder, reqs), eng.config.mtp_heads, steps)
    assert eng.free_pages() == eng.total_pages()


@pytest.mark.parametrize("backend", backends())
@pytest.mark.parametrize("name,dtype", CASES)
def test_portions_of_changing_size(name, dtype, backend):
    reqs = requests_for(name, [97, 50], seed=3)
    folder, eng = make_engine(name, dtype, backend, max_tokens=128)
    steps = H.portions_trace(reqs, seed=1)
    main, heads = H.run_trace(eng, steps)
    H.compare_with_plain(folder, reqs, main, heads, TOL[dtype] * scale_of(folder, reqs), eng.config.mtp_heads, steps)
    assert eng.free_pages() == eng.total_pages()


@pytest.mark.parametrize("backend", backends())
@pytest.mark.parametrize("name,dtype", CASES)
def test_mixed_batches_with_page_reuse(name, dtype, backend):
    lengths = [50, 64, 37, 90, 18, 70, 45, 3, 66, 29]
    reqs = requests_for(name, lengths, seed=4)
    steps, peak = H.mixed_trace(reqs, max_live=4, seed=5)
    # so few pages that finished requests' pages must be handed out again
    folder, eng = make_engine(name, dtype, backend, max_tokens=peak)
    assert sum(-(-n // 64) * 64 for n in lengths) > 2 * peak
    main, heads = H.run_trace(eng, steps)
    H.compare_with_plain(folder, reqs, main, heads, TOL[dtype] * scale_of(folder, reqs), eng.config.mtp_heads, steps)
    eng.cache.check()
    assert eng.free_pages() == eng.total_pages()


@pytest.mark.parametrize("backend", backends())
@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("B", "bfloat16")])
def test_first_tokens_and_long_decoding(name, dtype, backend):
    """One token at a time from the very first position: the heads start late, every page edge is crossed."""
    n = 150 if name == "A" else 120
    reqs = requests_for(name, [n], seed=6)
    folder, eng = make_engine(name, dtype, backend, max_tokens=192)
    ids = reqs["r0"]
    steps = [{"step": p, "entries": [{"id": "r0", "tokens": [ids[p]], "want": [0]}],
              "end": ["r0"] if p == n - 1 else []} for p in range(n)]
    main, heads = H.run_trace(eng, steps)
    assert len(main) == n
    M = eng.config.mtp_heads
    for hi in range(M):
        assert all(("r0", hi, p) in heads for p in range(n - 1 - hi))
    H.compare_with_plain(folder, reqs, main, heads, TOL[dtype] * scale_of(folder, reqs), M, steps)


@pytest.mark.parametrize("backend", backends())
def test_all_schedules_agree_with_each_other(backend):
    """The same (request, position) under four schedules: differences stay within rounding of 32-bit sums."""
    name, dtype = "B", "float32"
    reqs = requests_for(name, [61, 44], seed=7)
    outs = []
    for trace in (H.whole_trace(reqs), H.tail_decode_trace(reqs, 32), H.portions_trace(reqs, 2),
                  H.mixed_trace(reqs, 2, 3)[0]):
        folder, eng = make_engine(name, dtype, backend, max_tokens=128)
        outs.append(H.run_trace(eng, trace)[0])
    for other in outs[1:]:
        assert other.keys() == outs[0].keys()
        worst = max((other[k] - outs[0][k]).abs().max().item() for k in other)
        assert worst <= 2e-5


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["B", "C", "D"])
def test_schedules_with_portions_on_the_tile_kernel(name, monkeypatch):
    """Beside decoded tokens deep in their requests the tiny models' portions are too little work for the workgroup
    attention kernel to be chosen; here it is made to take every portion that fills half a tile, and whole prompts,
    portions and mixed batches (with pages handed out again) are compared with the plain implementation as elsewhere."""
    from tiny_inference_server_amd.ops import hip_ops
    monkeypatch.setattr(hip_ops, "_ATTN_TILE_MIN_WORK_MIXED", 0)
    planned = {"tiles": 0}
    plan = hip_ops.attention_items

    def counting(*args, **kw):
        out = plan(*args, **kw)
        planned["tiles"] += len(out[2])
        return out
    monkeypatch.setattr(hip_ops, "attention_items", counting)
    lengths = [97, 50, 64, 37, 90, 18, 70]
    reqs = requests_for(name, lengths, seed=8)
    mixed, peak = H.mixed_trace(reqs, max_live=4, seed=6)
    for trace, max_tokens in ((H.whole_trace(reqs), 512), (H.portions_trace(reqs, seed=4), 512), (mixed, peak)):
        folder, eng = make_engine(name, "bfloat16", "hip", max_tokens=max_tokens)
        main, heads = H.run_trace(eng, trace)
        assert planned["tiles"] > 0          # whole prompts always fill tiles; the short portions of C may not
        H.compare_with_plain(folder, reqs, main, heads, TOL["bfloat16"] * scale_of(folder, reqs), eng.config.mtp_heads,
                             trace)
        eng.cache.check()
        assert eng.free_pages() == eng.total_pages()


@pytest.mark.gpu
def test_long_context_decoding_in_bfloat16():
    """A prompt of 500 tokens in uneven portions, then 120 tokens one by one through captured graphs: keys are cut
    into several splits, pages are crossed, and every logit still matches the plain model."""
    name, dtype = "D", "bfloat16"
    reqs = requests_for(name, [620], seed=8)
    folder, eng = make_engine(name, dtype, "hip", max_tokens=640)
    ids = reqs["r0"]
    steps, p = [], 0
    for n in [333, 100, 67] + [1] * 120:
        steps.append({"step": len(steps), "entries": [{"id": "r0", "tokens": ids[p:p + n], "want": [n - 1] if n > 1 else [0]}],
                      "end": []})
        p += n
    main, _ = H.run_trace(eng, steps, heads=False)
    assert eng.graph_replays >= 100
    H.compare_with_plain(folder, reqs, main, {}, TOL[dtype] * scale_of(folder, reqs), 0, steps)


@pytest.mark.parametrize("backend", backends())
@pytest.mark.parametrize("seed", [11, 12, 13, 14])
@pytest.mark.parametrize("name,dtype", [("B", "float32"), ("D", "bfloat16")])
def test_random_schedules(name, dtype, backend, seed):
    """Request lengths, the number of live requests, where prompts end and how they are cut all drawn at random, on
    a pool just large enough: whatever the schedule, the logits are the plain model's."""
    import random
    rng = random.Random(seed)
    lengths = [rng.choice((1, 2, 3, 15, 16, 17, 31, 32, 33, 47, 63, 64, 65, 80, 100)) for _ in range(rng.randint(5, 9))]
    reqs = requests_for(name, lengths, seed=seed)
    steps, peak = H.mixed_trace(reqs, max_live=rng.randint(1, 4), seed=seed, prompt_frac=rng.choice((0.0, 0.3, 0.7, 1.0)))
    folder, eng = make_engine(name, dtype, backend, max_tokens=peak)
    main, heads = H.run_trace(eng, steps)
    H.compare_with_plain(folder, reqs, main, heads, TOL[dtype] * scale_of(folder, reqs), eng.config.mtp_heads, steps)
    eng.cache.check()
    assert eng.free_pages() == eng.total_pages()


def drawn_configuration(seed):
    """A tiny configuration with every size drawn: heads and groups (also groups that do not divide a wave's columns),
    head sizes in steps of 8 (those in steps of 16 run on the matrix cores, the others on the general kernel), widths
    and vocabularies that are no power of two, layers, prediction heads, the norms' eps, the rotary base, the page."""
    import random
    from tiny_inference_server_amd.config import GqaMtpConfig
    rng = random.Random(1000 + seed)
    n_kv, group = rng.choice([1, 1, 2, 3, 4]), rng.choice([1, 2, 3, 4, 5, 8])
    hd = rng.choice([16, 32, 48, 64, 80, 96, 128, 8, 24, 40])
    while n_kv * group * hd > 1280:
        n_kv, group = max(1, n_kv - 1), max(1, group - 1)
    cfg = GqaMtpConfig(d_model=n_kv * group * hd, vocab_size=rng.choice([97, 300, 515, 1000, 2049, 3001]),
                       max_context=rng.choice([200, 320, 512]), rope_base=rng.choice([1000.0, 10000.0, 500000.0]),
                       n_heads=n_kv * group, n_layers=rng.randint(1, 3),
                       ffn_hidden=rng.choice([88, 176, 200, 264, 320, 520, 1000, 1408]), group_size=group,
                       mtp_heads=rng.randint(0, 2), rms_eps=rng.choice([2e-8, 1e-6, 1e-5]),
                       tie_embeddings=rng.random() < 0.5)
    wide = dict(std=0.02, sharpen=2.0) if cfg.d_model >= 512 else {}
    return rng, dict(cfg=cfg, page_size=rng.choice([8, 16, 16, 32]), gain_jitter=0.1, seed=100 + seed, **wide)


@pytest.mark.parametrize("seed,backend", [pytest.param(s, "hip", marks=pytest.mark.gpu) for s in range(24)]
                         + [(s, "torch") for s in (0, 3, 29)])
def test_drawn_configurations_under_drawn_schedules(seed, backend):
    """Not the few configurations the other tests know: every size of the model drawn at random, then a precision and
    a family of schedules drawn too, against the plain implementation at the fixed tolerances."""
    name = f"drawn{seed}"
    rng, H.TINY[name] = drawn_configuration(seed)
    cfg = H.TINY[name]["cfg"]
    dtype = rng.choice(["bfloat16", "bfloat16", "float32"])
    kind = rng.choice(["whole", "tail", "portions", "mixed", "mixed"])
    lengths = [rng.randint(1, min(150, cfg.max_context - 4)) for _ in range(rng.randint(2, 7))]
    reqs = requests_for(name, lengths, seed=seed)
    steps, peak = {"whole": lambda: (H.whole_trace(reqs), 256), "tail": lambda: (H.tail_decode_trace(reqs, 32), 256),
                   "portions": lambda: (H.portions_trace(reqs, seed=seed), 256),
                   "mixed": lambda: H.mixed_trace(reqs, max_live=4, seed=seed)}[kind]()
    folder, eng = make_engine(name, dtype, backend, max_tokens=max(peak, 64))
    main, heads = H.run_trace(eng, steps)
    H.compare_with_plain(folder, reqs, main, heads, TOL[dtype] * scale_of(folder, reqs), cfg.mtp_heads, steps)
    eng.cache.check()
    assert eng.free_pages() == eng.total_pages()


@pytest.mark.gpu
@pytest.mark.parametrize("seed", range(16))
def test_drawn_configurations_decoding_together_through_captured_steps(seed):
    """Drawn sizes again, now for the steps that serving is made of: one to twenty requests' prompts (half of the
    time most of them short beside a few long ones, so that splits are planned request by request), then all of them
    decoding together for up to thirty steps, which are captured and replayed (more than eight requests: the shapes
    with filler lines); one request may end early, so that the step's shape changes under way. Every page starts out
    full of NaN. The first stage's logits against the plain implementation."""
    import random
    name = f"together{seed}"
    rng, H.TINY[name] = drawn_configuration(seed + 500)
    cfg = H.TINY[name]["cfg"]
    dtype = rng.choice(["bfloat16", "bfloat16", "float32"])
    n_req, n_dec, uneven = rng.choice([1, 2, 3, 5, 8, 9, 12, 17, 20]), rng.randint(8, 30), rng.random() < 0.5
    lens = [rng.randint(cfg.mtp_heads + 3, 20 if (uneven and i % 3) else min(150, cfg.max_context - n_dec - 4))
            for i in range(n_req)]
    reqs = {f"r{i}": H.random_ids(cfg.vocab_size, n + n_dec, seed * 100 + i) for i, n in enumerate(lens)}
    steps = [{"step": i, "entries": [{"id": rid, "tokens": ids[:lens[i]], "want": [lens[i] - 1]}], "end": []}
             for i, (rid, ids) in enumerate(reqs.items())]
    leave = rng.choice([None, rng.randint(2, n_dec - 2)]) if n_req > 2 else None      # the step after which r1 is gone
    for k in range(n_dec):
        live = [(i, rid) for i, rid in enumerate(reqs) if not (leave is not None and i == 1 and k >= leave)]
        ended = (["r1"] if leave is not None and k == leave - 1 else []) + ([rid for _, rid in live] if k == n_dec - 1 else [])
        steps.append({"step": len(steps), "end": ended,
                      "entries": [{"id": rid, "tokens": [reqs[rid][lens[i] + k]], "want": [0]} for i, rid in live]})
    if leave is not None:
        reqs["r1"] = reqs["r1"][:lens[1] + leave]
    folder, eng = make_engine(name, dtype, "hip", max_tokens=sum(-(-len(v) // 64) * 64 for v in reqs.values()),
                              max_requests=max(4, n_req))
    H.fill_cache_with_nan(eng)
    main, _ = H.run_trace(eng, steps, heads=False)
    assert eng.graph_replays >= n_dec // 2
    H.compare_with_plain(folder, reqs, main, {}, TOL[dtype] * scale_of(folder, reqs), 0)
    eng.cache.check()
    assert eng.free_pages() == eng.total_pages()


@pytest.mark.parametrize("backend", backends())
@pytest.mark.parametrize("name,dtype", [("D", "bfloat16"), ("B", "float32")])
def test_what_a_page_held_before_never_reaches_a_result(name, dtype, backend):
    """Every page starts out full of NaN, as if a broken request had owned it: masked slots are read by the kernels
    but must not enter their arithmetic, not even weighted by zero."""
    lengths = [50, 64, 37, 90, 18, 70]
    reqs = requests_for(name, lengths, seed=8)
    steps, peak = H.mixed_trace(reqs, max_live=3, seed=9)
    folder, eng = make_engine(name, dtype, backend, max_tokens=peak)
    for g in eng.cache.groups.values():
        g.storage.fill_(float("nan"))
    main, heads = H.run_trace(eng, steps)
    H.compare_with_plain(folder, reqs, main, heads, TOL[dtype] * scale_of(folder, reqs), eng.config.mtp_heads, steps)


@pytest.mark.parametrize("name,dtype,backend", BIG_CASES)
def test_schedule_families_at_model_geometries(name, dtype, backend):
    """Whole prompts, prompt then decoding one by one, portions of changing size, and mixed batches on few pages, at
    the headline model's layer sizes (E: 12 query heads of 128 over 3 key/value heads) and at the attention
    geometries of the larger sizes (F: 16 over 4, G: 32 over 8): the matrix-core kernels with a group of four, several
    key/value heads, the few-row products at these widths. Nothing is patched; the planner chooses as it does in use."""
    reqs = requests_for(name, [5, 33, 70, 90, 47, 18], seed=21)
    mixed, peak = H.mixed_trace(reqs, max_live=4, seed=22)
    for steps, max_tokens in ((H.whole_trace(reqs), 128), (H.tail_decode_trace(reqs, tail=32), 128),
                              (H.portions_trace(reqs, seed=3), 128), (mixed, peak)):
        folder, eng = make_engine(name, dtype, backend, max_tokens=max_tokens)
        main, heads = H.run_trace(eng, steps)
        H.compare_with_plain(folder, reqs, main, heads, TOL[dtype] * scale_of(folder, reqs), eng.config.mtp_heads, steps)
        eng.cache.check()
        assert eng.free_pages() == eng.total_pages()


@pytest.mark.gpu
@pytest.mark.parametrize("name,cut", [("E", (1600, 448)), ("F", (1296, 200)), ("G", (900, 100))])
def test_long_prompt_cut_in_two_at_model_geometries(name, cut, monkeypatch):
    """A long prompt in two portions, then a few tokens one by one. The first portion is long enough for the planner
    to give it to the workgroup (tile) attention kernel at its real thresholds and to the sixteen-row rotary kernel;
    the second runs behind it over the paged context, its key ranges split and merged; the prediction heads run
    their shifted rows. Every position's main and head logits are compared with the plain implementation."""
    from tiny_inference_server_amd.ops import hip_ops
    planned = {"tiles": 0, "items": 0}
    plan = hip_ops.attention_items

    def counting(*args, **kw):
        out = plan(*args, **kw)
        planned["items"] += len(out[1])
        planned["tiles"] += len(out[2])
        return out
    monkeypatch.setattr(hip_ops, "attention_items", counting)
    n = sum(cut) + 4
    reqs = requests_for(name, [n], seed=23)
    ids = reqs["r0"]
    folder, eng = make_engine(name, "bfloat16", "hip", max_tokens=-(-n // 64) * 64)
    steps, p = [], 0
    for k in list(cut) + [1] * 4:
        steps.append({"step": len(steps), "entries": [{"id": "r0", "tokens": ids[p:p + k], "want": list(range(k))}],
                      "end": ["r0"] if p + k == n else []})
        p += k
    main, heads = H.run_trace(eng, steps)
    assert planned["tiles"] > 0 and planned["items"] > 0
    H.compare_with_plain(folder, reqs, main, heads, TOL["bfloat16"] * scale_of(folder, reqs), eng.config.mtp_heads, steps)
    assert eng.free_pages() == eng.total_pages()


@pytest.mark.parametrize("backend", backends())
@pytest.mark.parametrize("name,dtype", [("B", "float32"), ("D", "bfloat16")])
def test_first_stage_logits_do_not_depend_on_asking_for_the_heads(name, dtype, backend):
    """A step that also asks for the prediction heads' logits makes one product with the output table for all stages;
    a step that does not, one for the first stage alone. Both go through the same gather and the same product on the
    same rounded operands; only the order of a row's 32-bit partial sums may differ with the number of rows (the
    few-row kernel cuts K differently for up to 8 rows), so the first stage's logits agree to 32-bit rounding."""
    reqs = requests_for(name, [23, 40, 9], seed=9)
    outs = []
    for heads in (True, False):
        folder, eng = make_engine(name, dtype, backend, max_tokens=256)
        got = []
        for rid, ids in reqs.items():
            got.append(eng.step([(rid, ids[:-3], list(range(len(ids) - 3)))], heads=heads).logits.clone())
        for k in range(3, 0, -1):       # single tokens, all requests in one step
            got.append(eng.step([(rid, [ids[-k]], [0]) for rid, ids in reqs.items()], heads=heads).logits.clone())
        outs.append(got)
    for a, b in zip(*outs):
        # (in bfloat16 the two steps may also differ upstream of the product: a step of single tokens that asks for
        # the first stage alone is replayed from a captured graph, whose attention cuts its keys for the graph's width)
        torch.testing.assert_close(a, b, rtol=1e-5, atol=1e-4 if dtype == "float32" else 5e-2)

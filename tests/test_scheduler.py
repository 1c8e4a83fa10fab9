"""The scheduler's decisions, on the CPU with the torch stand-ins for the kernels: admission plans, portions
under a token budget, preemption and replay, finishing, pages given back."""
import pytest
import torch

import helpers as H
import plain_model as pm
from torch_ops import TorchOps
from tiny_inference_server_amd.engine import Engine
from tiny_inference_server_amd.engine.generate import generate
from tiny_inference_server_amd.engine.scheduler import Request, Scheduler, pages_for
from tiny_inference_server_amd.sampling import SamplingParams, uniform_for

NAME = "A"
LENS = [7, 33, 18, 1, 2]          # the reference's ragged prompts, with lengths 1 and 2 (test_server.py:69)


def engine(pool_tokens, max_requests=8, name=NAME):
    return Engine(H.model_folder(name, "float32"), dtype="float32", page_size=H.TINY[name]["page_size"],
                  max_tokens=pool_tokens, max_requests=max_requests, ops=TorchOps())


def prompts(name=NAME, lens=LENS):
    v = H.TINY[name]["cfg"].vocab_size
    return [H.random_ids(v, n, 80 + i) for i, n in enumerate(lens)]


@pytest.fixture(scope="module")
def greedy_truth():
    cfg, w = pm.read_model_folder(H.model_folder(NAME, "float32"))
    return [pm.greedy_generate(p, 20, w, cfg) for p in prompts()]


def test_greedy_equals_plain_and_pool_drains(greedy_truth):
    eng = engine(1024)
    out, s = generate(eng, prompts(), max_new_tokens=20, temperature=0.0, return_scheduler=True)
    assert out == greedy_truth
    assert s.preempts == 0 and eng.free_pages() == eng.total_pages() and eng.cache.n_live == 0


def test_forced_preemption_gives_the_same_tokens(greedy_truth):
    """The reference's check (test_server.py:114-118): a pool of a few pages, 2 slots, plan 'cur' -> preemption
    fires, greedy output is unchanged, every page comes back."""
    eng = engine(5 * 16, max_requests=2)
    out, s = generate(eng, prompts(), max_new_tokens=20, temperature=0.0, max_batch=2, token_budget=64, plan="cur",
                      return_scheduler=True)
    assert out == greedy_truth
    assert s.preempts >= 1 and s.replays >= 1
    assert eng.free_pages() == eng.total_pages() == 5


def test_plan_final_never_preempts(greedy_truth):
    eng = engine(5 * 16, max_requests=4)
    out, s = generate(eng, prompts(), max_new_tokens=20, temperature=0.0, max_batch=4, plan="final", return_scheduler=True)
    assert out == greedy_truth and s.preempts == 0
    assert s.peak_running <= 3          # 5 pages cannot hold four requests at full length


def test_admission_budget_counts_what_was_just_admitted():
    """Pages are only taken when a request runs; admission must not let the whole queue in on one free count
    (the reference's fix: server.py:143-147)."""
    eng = engine(4 * 16, max_requests=8)
    s = Scheduler(eng, max_batch=8, token_budget=256, plan="cur")
    for p in prompts(lens=[30, 30, 30, 30]):
        s.submit(Request(p, SamplingParams(max_new_tokens=4, temperature=0.0)))
    s.admit()
    assert len(s.active) == 2 and len(s.queue) == 2       # 2 pages each: two fit in 4 pages
    s.step()
    assert s.preempts == 0


def test_token_budget_cuts_prompts_into_portions_beside_decodes():
    eng = engine(1024)
    s = Scheduler(eng, max_batch=4, token_budget=12, plan="final")
    a, b = Request(prompts()[0], SamplingParams(max_new_tokens=30, temperature=0.0)), \
        Request(prompts()[1], SamplingParams(max_new_tokens=3, temperature=0.0))
    s.submit(a)
    s.admit(); s.step()                                   # a: 7 prompt tokens at once, first token sampled
    assert a.fed == 7 and len(a.ids) == 8
    s.submit(b)
    s.admit()
    plan = s.plan_step()
    assert [(r.id, start, n, smp) for r, start, n, smp in plan.items] == [(a.id, 7, 1, True), (b.id, 0, 11, False)]
    s.step()
    assert b.fed == 11 and len(b.ids) == 33 and len(a.ids) == 9
    s.step(); s.step()
    assert b.fed == 33 and len(b.ids) == 34               # the portion that ends the prompt samples its first token
    fin = s.run()
    assert {r.id for r in fin} == {a.id, b.id} and len(b.out_ids()) == 3 and len(a.out_ids()) == 30


def test_portions_do_not_change_the_tokens(greedy_truth):
    for budget in (8, 13, 40):
        out = generate(engine(1024), prompts(), max_new_tokens=10, temperature=0.0, max_batch=8, token_budget=budget)
        assert out == [t[:10] for t in greedy_truth], budget


def test_a_lone_request_that_cannot_fit_is_an_error():
    eng = engine(2 * 16, max_requests=2)
    with pytest.raises(RuntimeError, match="kv pool too small for a single request"):
        generate(eng, [H.random_ids(512, 40, 1)], max_new_tokens=4, temperature=0.0)
    with pytest.raises(ValueError, match="leaves no room"):
        Scheduler(engine(1024)).submit(Request(H.random_ids(512, 256, 2)))


def test_finishing_rules():
    """End-of-sequence token, max_new_tokens, the model's context (reference server.py:242-252)."""
    cfg, w = pm.read_model_folder(H.model_folder(NAME, "float32"))
    p = prompts()[0]
    free = pm.greedy_generate(p, 6, w, cfg)
    eng = engine(1024)
    eng.spec = type(eng.spec)(**{**eng.spec.__dict__, "eos_token_id": free[2]})
    out = generate(eng, [p], max_new_tokens=6, temperature=0.0)
    assert out == [free[:free.index(free[2]) + 1]]        # cut after the first end token, which is kept
    eng2 = engine(1024)
    eng2.spec = eng.spec
    out = generate(eng2, [p], max_new_tokens=6, temperature=0.0, ignore_eos=True)
    assert out == [free]
    long_prompt = H.random_ids(512, 250, 3)
    out, s = generate(engine(1024), [long_prompt], max_new_tokens=50, temperature=0.0, return_scheduler=True)
    assert len(out[0]) == 256 - 250                       # stops at the model's context of 256


def test_sampled_tokens_do_not_depend_on_the_batch():
    """Each request has its own random stream, so alone or batched, preempted or not, it draws the same tokens."""
    ps = prompts()
    params = [SamplingParams(max_new_tokens=20, temperature=0.8, top_k=20, top_p=0.9, rep_penalty=1.2, seed=100 + i)
              for i in range(len(ps))]
    together = generate(engine(1024), ps, params=params, max_batch=8)
    alone = [generate(engine(1024), [p], params=[sp])[0] for p, sp in zip(ps, params)]
    squeezed, s = generate(engine(5 * 16, max_requests=2), ps, params=params, max_batch=2, plan="cur", token_budget=16,
                           return_scheduler=True)
    assert together == alone == squeezed and s.preempts >= 1
    other = generate(engine(1024), ps, params=[SamplingParams(**{**sp.__dict__, "seed": sp.seed + 1}) for sp in params])
    assert other != together


def test_temperature_sampling_matches_the_plain_rule():
    """Token by token: the plain model's probabilities (server.py:22-50) and the same uniform number give the
    engine's token."""
    cfg, w = pm.read_model_folder(H.model_folder(NAME, "float32"))
    p = prompts()[2]
    sp = SamplingParams(max_new_tokens=6, temperature=0.8, top_k=30, top_p=0.9, rep_penalty=1.3, seed=5)
    got = generate(engine(1024), [p], params=[sp])[0]
    ids = list(p)
    for i in range(6):
        lg = pm.logits_of(pm.trunk_hidden(ids, w, cfg)[-1:], w, cfg)[0]
        probs = pm.sampling_probs(lg, sp.temperature, sp.top_k, sp.top_p, sp.rep_penalty, ids)
        ids.append(pm.pick_by_uniform(probs, uniform_for(sp.seed, i)))
    assert got == ids[len(p):]


def test_uniform_stream():
    u = [uniform_for(3, i) for i in range(2000)]
    assert all(0.0 <= x < 1.0 for x in u) and len(set(u)) > 1990
    assert abs(sum(u) / len(u) - 0.5) < 0.03
    assert uniform_for(3, 7) == uniform_for(3, 7) != uniform_for(4, 7)


def test_pages_for():
    assert [pages_for(n, 16) for n in (0, 1, 16, 17)] == [0, 1, 1, 2]


@pytest.mark.parametrize("static", ["req", 64, "ctx"])
def test_static_modes_take_pages_at_admission_and_give_the_same_tokens(greedy_truth, static):
    """The reference's storage policy static="ctx"/"req"/<int> (server.py:107-111, 151-166, 180-185): every page of
    a request is taken when it is admitted, nothing is preempted, the tokens are the paged ones."""
    eng = engine(16 * 64, max_requests=4)
    s = Scheduler(eng, max_batch=4, token_budget=64, plan="cur", static=static,
                  max_context=128 if static == "ctx" else None)
    reqs = [Request(p, SamplingParams(max_new_tokens=20, temperature=0.0)) for p in prompts()]
    for r in reqs:
        s.submit(r)
    s.admit()
    want_pages = {"req": lambda r: pages_for(r.prompt_len + 20, 16), 64: lambda r: 4, "ctx": lambda r: 8}[static]
    assert s.active and all(r.reserved == want_pages(r) * 16 for r in s.active)
    assert eng.total_pages() - eng.free_pages() == sum(want_pages(r) for r in s.active)       # taken before any step
    s.run()
    assert [r.out_ids() for r in reqs] == greedy_truth
    assert s.preempts == 0 and eng.free_pages() == eng.total_pages() and eng.cache.n_live == 0


def test_static_reservation_larger_than_the_pool_is_an_error():
    eng = engine(2 * 16, max_requests=2)
    s = Scheduler(eng, max_batch=2, static=64)
    s.submit(Request(prompts()[0], SamplingParams(max_new_tokens=4, temperature=0.0)))
    with pytest.raises(RuntimeError, match="static reservation 4 pages > pool 2"):
        s.admit()


def test_static_admission_waits_for_pages_instead_of_preempting(greedy_truth):
    """Six pages, every request reserves two or three: they run two at a time, and none is thrown out."""
    eng = engine(6 * 16, max_requests=4)
    out, s = generate(eng, prompts(), max_new_tokens=20, temperature=0.0, max_batch=4, plan="cur", static="req",
                      return_scheduler=True)
    assert out == greedy_truth and s.preempts == 0 and s.peak_running <= 3
    assert eng.free_pages() == eng.total_pages() == 6


def test_twelve_sampled_requests_with_heads_on_a_pool_of_nan_through_kept_steps():
    """The GPU suite's schedule at the headline geometry, here in 32-bit on the stand-in with kept steps emulated, so
    that the host side alone is on trial: more live requests than captured steps have exact shapes for (filler lines),
    the prediction heads run, plan "cur" preempts, sampling with temperature and repetition penalty from per-request
    streams, pages full of NaN beforehand. Every token is the reference rule's draw on the plain model's logits."""
    name, n_req = "A", 12
    folder = H.model_folder(name, "float32")
    prompts, params = H.sampled_workload(name, n_req, seed=310, temperature=0.7, rep_penalty=1.3)
    eng = Engine(folder, dtype="float32", page_size=16, max_tokens=40 * 16, max_requests=n_req,
                 ops=TorchOps(graphs=True), run_heads=True)
    H.fill_cache_with_nan(eng)
    steps = H.watch_decode_steps(eng)
    s = Scheduler(eng, max_batch=n_req, token_budget=64, plan="cur")
    reqs = [Request(p, sp) for p, sp in zip(prompts, params)]
    for r in reqs:
        s.submit(r)
    s.run()
    assert s.preempts > 0 and s.replays > 0
    assert any(n > 8 and n % 8 and replayed for n, replayed in steps), steps
    checked, equal = H.check_sampled_tokens(folder, prompts, params, [r.out_ids() for r in reqs], slack=1e-5)
    assert checked == sum(sp.max_new_tokens for sp in params) and equal >= checked - 2, (checked, equal)
    eng.cache.check()
    assert eng.free_pages() == eng.total_pages() and eng.cache.n_live == 0

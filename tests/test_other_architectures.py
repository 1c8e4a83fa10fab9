"""What a model of another architecture needs from the host side, shown with toy models defined in the tests and the
torch stand-ins for the kernels: a model whose mixers keep state of fixed size only (no pages at all) and a model whose
layers all see a window go through the scheduler and generate() without a change to the framework's files."""
import dataclasses

import pytest
import torch

import helpers as H
import plain_model as pm
from torch_ops import TorchOps
from toy_parts import ToyConfig, ToyDecayMixer, toy_plain, toy_spec
from tiny_inference_server_amd.cache import CacheManager
from tiny_inference_server_amd.config import ARCHITECTURES, Architecture, GqaMtpConfig
from tiny_inference_server_amd.engine import Engine
from tiny_inference_server_amd.engine.generate import generate
from tiny_inference_server_amd.engine.scheduler import Request, Scheduler
from tiny_inference_server_amd.parts import MIXERS, LayerCall, ModelSpec, PartSpec, StageSpec
from tiny_inference_server_amd.sampling import SamplingParams
from tiny_inference_server_amd.weights import random_tensors


@pytest.fixture
def toy_state_model():
    ARCHITECTURES.register("ToyStateModel", Architecture("ToyStateModel", ToyConfig, toy_spec), replace=True)
    MIXERS.register("toy_decay", ToyDecayMixer, replace=True)
    cfg = ToyConfig(d_model=48, vocab_size=101, hidden=80, decay=0.7)
    w = random_tensors(cfg, 9, std=0.1, gain_jitter=0.1, dtype="float32")
    yield cfg, w
    ARCHITECTURES.unregister("ToyStateModel")
    MIXERS.unregister("toy_decay")


def toy_greedy(prompt, n_new, w, cfg):
    ids = list(prompt)
    for _ in range(n_new):
        ids.append(int(torch.argmax(toy_plain(ids, w, cfg)[-1])))
    return ids[len(prompt):]


@pytest.mark.parametrize("plan,max_batch", [("final", 2), ("cur", 3)])
def test_a_model_without_pages_generates_through_the_scheduler(toy_state_model, plan, max_batch):
    """No mixer of this model keeps keys and values: the cache manager has no page group, pages never run out, and
    admission is bounded by the request slots alone."""
    cfg, w = toy_state_model
    eng = Engine(config=cfg, tensors=w, dtype="float32", max_requests=max_batch, ops=TorchOps())
    assert not eng.cache.groups and eng.free_pages() == eng.total_pages() == Engine.NO_PAGE_LIMIT
    assert eng.pages_to_hold(1000, 64) == 0
    prompts = [H.random_ids(101, n, 30 + i) for i, n in enumerate((13, 1, 7, 22))]
    out, s = generate(eng, prompts, max_new_tokens=6, temperature=0.0, max_batch=max_batch, token_budget=9, plan=plan,
                      return_scheduler=True)
    assert out == [toy_greedy(p, 6, w, cfg) for p in prompts]
    assert s.preempts == 0 and s.peak_running == max_batch and eng.cache.n_live == 0
    eng.cache.check()


def windowed_spec(cfg, windows):
    from tiny_inference_server_amd.architectures.gqa_mtp import _block, _norm
    layers = []
    for l, win in enumerate(windows):
        blk = _block(cfg, f"transformer_block_list.{l}.")
        mixer = blk.part("mixer")
        layers.append(blk.with_part("mixer", dataclasses.replace(mixer, params={**mixer.params, "window": win})))
    stage = StageSpec("trunk", 0, PartSpec("stage_input", "token_embedding"), tuple(LayerCall(l) for l in range(len(windows))),
                      _norm(cfg, "rms_out.scale"))
    return ModelSpec(cfg.d_model, cfg.vocab_size, cfg.max_context, tuple(layers), (stage,), "embedding.weight", "embedding.weight")


def windowed_greedy(prompt, n_new, w64, cfg, windows):
    ids = list(prompt)
    pcfg = {"n_heads": cfg.n_heads, "group": cfg.group_size, "eps": cfg.rms_eps, "base": cfg.rope_base}
    for _ in range(n_new):
        x = w64["embedding.weight"][torch.tensor(ids)]
        for l, win in enumerate(windows):
            x = pm.block(x, w64, f"transformer_block_list.{l}.", pcfg, torch.arange(len(ids)), window=win)
        ids.append(int(torch.argmax(pm.rms_norm(x[-1:], w64["rms_out.scale"], cfg.rms_eps) @ w64["embedding.weight"].T)))
    return ids[len(prompt):]


def test_a_model_of_windows_alone_is_planned_by_what_its_windows_hold():
    """Both layers see a window, so a request never holds more than a window's pages and a step's. The scheduler asks
    the engine what a request holds instead of counting a page for every 8 tokens: two requests that would need 24
    pages by that count run side by side, to the end, in a pool of 18, with no preemption."""
    windows = (24, 40)
    cfg = GqaMtpConfig(d_model=64, vocab_size=97, max_context=256, rope_base=1e4, n_heads=4, n_layers=2, ffn_hidden=96,
                       group_size=2, mtp_heads=0, architecture="WindowsOnly")
    ARCHITECTURES.register("WindowsOnly", Architecture("WindowsOnly", GqaMtpConfig, lambda c: windowed_spec(c, windows)),
                           replace=True)
    try:
        w = random_tensors(cfg, 23, std=0.08, gain_jitter=0.1, dtype="float32")
        eng = Engine(config=cfg, tensors=w, dtype="float32", page_size=8, n_pages=18, max_requests=2, ops=TorchOps())
        assert sorted(eng.cache.groups) == ["kv2x16w24", "kv2x16w40"]
        # a window of 40, portions of at most 8 tokens, pages of 8: ceil(48 / 8) + 1 pages at a time, however long
        assert eng.pages_to_hold(100, 8) == 7 and eng.pages_to_hold(30, 8) == 4 and eng.pages_to_hold(100, 100) == 13
        prompts = [H.random_ids(97, 60, 51), H.random_ids(97, 45, 52)]
        out, s = generate(eng, prompts, max_new_tokens=40, temperature=0.0, max_batch=2, token_budget=8, plan="final",
                          return_scheduler=True)
        w64 = {k: v.double() for k, v in w.items()}
        assert out == [windowed_greedy(p, 40, w64, cfg, windows) for p in prompts]
        assert s.preempts == 0 and s.peak_running == 2
        eng.cache.check()
        assert eng.free_pages() == eng.total_pages() == 18
        # by a page for every 8 tokens the two would have needed 13 + 11 pages: the same pool, planned that way,
        # would have run them one after the other
        assert -(-100 // 8) + -(-85 // 8) > 18
    finally:
        ARCHITECTURES.unregister("WindowsOnly")


def test_page_bytes_follow_the_parts_needs():
    from tiny_inference_server_amd.parts import PagedKvNeed, StateNeed
    needs = {"a": PagedKvNeed(2, 16), "b": PagedKvNeed(2, 16), "c": PagedKvNeed(1, 64, window=32), "s": StateNeed((8,))}
    assert CacheManager.page_bytes(needs, 16, torch.bfloat16) == (2 * 2 * 2 * 16 * 16 + 2 * 1 * 64 * 16) * 2
    assert CacheManager.page_bytes({"s": StateNeed((8,))}, 16, torch.float32) == 0
    m = CacheManager(needs, 16, 4, 2, torch.bfloat16, "cpu", allocate=False)
    assert m.bytes_per_position() == (2 * 2 * 2 * 16 + 2 * 1 * 64) * 2


def test_prediction_stage_takes_any_norm_on_its_embedding():
    """The stage that fuses the previous stage's output with the next token's embedding calls its norm through the
    interface every norm has (rows in, rows out), and fuses it into the gather only if the norm offers (gain, eps)."""
    from tiny_inference_server_amd.parts import NORMS
    from tiny_inference_server_amd.architectures.gqa_mtp import build_spec

    @NORMS.register("toy_center", replace=True)
    class ToyCenter:
        """y = (x - mean(x)) * gain: no (gain, eps) to hand to a fused kernel."""
        graph_safe = True

        @classmethod
        def tensor_shapes(cls, params):
            return {"gain": (params["width"],)}

        def __init__(self, spec, tensors, ops):
            self.gain = tensors.of(spec, "gain").float()

        def __call__(self, x):
            xf = x.float()
            return ((xf - xf.mean(-1, keepdim=True)) * self.gain).to(x.dtype)

    def spec_with_toy_norm(cfg):
        spec = build_spec(cfg)
        stages = list(spec.stages)
        st = stages[1]
        old = st.input.params["embed_norm"]
        new = PartSpec("norm", "toy_center", {"width": cfg.d_model}, dict(old.tensors))
        stages[1] = dataclasses.replace(st, input=dataclasses.replace(st.input, params={**st.input.params, "embed_norm": new}))
        return dataclasses.replace(spec, stages=tuple(stages))

    cfg = dataclasses.replace(H.TINY["A"]["cfg"], architecture="ToyNormHeads")
    ARCHITECTURES.register("ToyNormHeads", Architecture("ToyNormHeads", GqaMtpConfig, spec_with_toy_norm), replace=True)
    try:
        w = random_tensors(cfg, 5, std=0.05, gain_jitter=0.1, dtype="float32")
        eng = Engine(config=cfg, tensors=w, dtype="float32", page_size=16, max_tokens=128, max_requests=2, ops=TorchOps())
        ids = H.random_ids(cfg.vocab_size, 20, 3)
        out = eng.step([("a", ids, list(range(20)))], heads=True)
        w64 = {k: v.double() for k, v in w.items()}
        pc = _plain_cfg(cfg)
        h = pm.trunk_hidden(ids, w64, pc)
        torch.testing.assert_close(out.logits.double(), pm.logits_of(h, w64, pc), rtol=1e-4, atol=1e-5)
        # the plain head with the toy norm in place of the embedding's RMSNorm (reference main_models_new.py:163-171)
        e = w64["embedding.weight"][torch.tensor(ids[1:])]
        e = (e - e.mean(-1, keepdim=True)) * w64["mtp_heads_list.0.rms_embed.scale"]
        z = torch.cat((h[:-1], e), dim=-1) @ w64["mtp_heads_list.0.proj.weight"]
        z = pm.block(z, w64, "mtp_heads_list.0.trans_block.", pc, torch.arange(len(ids) - 1))
        want = pm.logits_of(pm.rms_norm(z, w64["mtp_heads_list.0.rms_out.scale"], cfg.rms_eps), w64, pc)
        got = out.head_logits[0]
        assert not out.head_valid[0][0]
        for row in range(1, 20):                 # the head's row p - 1 answers the wanted position p
            assert out.head_valid[0][row]
            torch.testing.assert_close(got[row].double(), want[row - 1], rtol=1e-4, atol=1e-5)
    finally:
        ARCHITECTURES.unregister("ToyNormHeads")
        NORMS.unregister("toy_center")


def _plain_cfg(cfg):
    return {"n_heads": cfg.n_heads, "group": cfg.group_size, "eps": cfg.rms_eps, "base": cfg.rope_base,
            "n_layers": cfg.n_layers, "mtp": cfg.mtp_heads, "tied": cfg.tie_embeddings, "vocab": cfg.vocab_size}

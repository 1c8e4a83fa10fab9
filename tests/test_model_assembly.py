"""How a model is put together from a spec, on the host: named parts of a block, cache keys for blocks with several
mixers, host planning found through the parts, graph promises, the run order as data. The kernels' stand-in runs the
steps; the run-order test also runs on the GPU."""
import dataclasses

import pytest
import torch

import helpers as H
import plain_model as pm
from tiny_inference_server_amd.architectures.gqa_mtp import build_spec
from tiny_inference_server_amd.config import GqaMtpConfig
from tiny_inference_server_amd.engine.model import Model
from tiny_inference_server_amd.parts import (ARRANGEMENTS, MIXERS, Arrangement, LayerCall, LayerSpec, ModelSpec, PagedKvNeed,
                                             PartSpec, StageSpec, StateNeed, to_compute)
from tiny_inference_server_amd.weights import random_tensors
from tiny_inference_server_amd.weights.loader import spec_tensors
from torch_ops import TorchOps

CFG = GqaMtpConfig(d_model=48, vocab_size=97, max_context=128, rope_base=1e4, n_heads=4, n_layers=2, ffn_hidden=40,
                   group_size=2, mtp_heads=1)


def test_a_block_is_an_arrangement_and_named_parts():
    spec = build_spec(CFG)
    blk = spec.layers[0]
    assert blk.arrangement == "prenorm_residual"
    assert set(blk.parts) == {"mixer_norm", "mixer", "feed_forward_norm", "feed_forward"}
    assert [n for n, _ in blk.mixers()] == ["mixer"]
    with pytest.raises(KeyError, match="has no part 'gate'.*feed_forward"):
        blk.part("gate")
    other = blk.with_part("mixer", dataclasses.replace(blk.part("mixer"), params={**blk.part("mixer").params, "window": 8}))
    assert other.part("mixer").params["window"] == 8 and blk.part("mixer").params.get("window", 0) == 0


def test_an_arrangement_refuses_parts_it_does_not_wire():
    spec = build_spec(CFG)
    w = random_tensors(CFG, 1, dtype="float32")
    blk = spec.layers[0]
    short = LayerSpec("prenorm_residual", {k: v for k, v in blk.parts.items() if k != "feed_forward"})
    with pytest.raises(ValueError, match="is made of .*feed_forward.* its spec brings"):
        Model(dataclasses.replace(spec, layers=(short,) + spec.layers[1:]), w, TorchOps())


class _Recurrence:
    """y = (decay * state + x) . W, state per request; promises graph safety for single rows only."""
    graph_safe = "single_rows"

    @classmethod
    def tensor_shapes(cls, params):
        return {"w": (params["d_model"], params["d_model"])}

    @classmethod
    def cache_need(cls, params):
        return StateNeed((params["d_model"],), "float32")

    def __init__(self, spec, tensors, ops):
        self.ops, self.w = ops, to_compute(ops, tensors.of(spec, "w").t())

    def forward(self, x, ctx, residual=None):
        return self.ops.linear(x, self.w, residual=residual)


class _Both(Arrangement):
    part_names = ("norm", "attention", "recurrence")

    def forward(self, x, ctx):
        a = self.parts["norm"](x)
        x = self.parts["attention"].forward(a, ctx.of("attention"), residual=x)
        return self.parts["recurrence"].forward(a, ctx.of("recurrence"), residual=x)


def test_every_mixer_of_a_block_gets_a_cache_of_its_own_and_planning_comes_from_the_parts():
    MIXERS.register("_recurrence", _Recurrence, replace=True)
    ARRANGEMENTS.register("_both", _Both, replace=True)
    try:
        base = build_spec(dataclasses.replace(CFG, mtp_heads=0))
        blk = base.layers[0]
        rec = PartSpec("mixer", "_recurrence", {"d_model": CFG.d_model}, {"w": "rec.w"})
        both = LayerSpec("_both", {"norm": blk.part("mixer_norm"), "attention": blk.part("mixer"), "recurrence": rec})
        stage = dataclasses.replace(base.stages[0], calls=(LayerCall(0), LayerCall(1), LayerCall(0, cache="again")))
        spec = dataclasses.replace(base, layers=(both, base.layers[1]), stages=(stage,))
        names = spec_tensors(spec)
        assert "rec.w" in names and not any(n.startswith("transformer_block_list.0.ffn") for n in names)
        w = {n: 0.1 * torch.randn(sh, generator=torch.Generator().manual_seed(i)) for i, (n, sh) in enumerate(sorted(names.items()))}
        model = Model(spec, w, TorchOps())
        needs = model.cache_needs()
        assert set(needs) == {"trunk.0:attention", "trunk.0:recurrence", "trunk.1", "again:attention", "again:recurrence"}
        assert isinstance(needs["trunk.0:recurrence"], StateNeed) and isinstance(needs["again:attention"], PagedKvNeed)
        assert model.graph_safe_single_rows and not model.graph_safe
        # the stand-in kernels plan nothing; operations that do are asked once per distinct attention shape
        assert model.plan_rows([(0, 0, 3)], lambda a: 0) == {}

        class Planning(TorchOps):
            def __init__(self):
                super().__init__()
                self.asked = []

            def plan_attention(self, n_heads, n_kv_heads, head_dim, seq_rows, add, mode=None, window=0):
                self.asked.append((n_heads, n_kv_heads, head_dim))
                return {("toy", n_heads): (add([1, 2, 3]), len(seq_rows))}

        ops = Planning()
        model = Model(spec, w, ops)
        got = model.plan_rows([(0, 0, 3), (3, 5, 1)], lambda a: 7)
        assert ops.asked == [(4, 2, 12)] and got == {("toy", 4): (7, 2)}      # three calls of two layers, one shape
    finally:
        MIXERS.unregister("_recurrence")
        ARRANGEMENTS.unregister("_both")


# ---- the run order is data: a layer that runs twice, and a layer that reads another layer's keys and values ----------

def run_order_spec(cfg):
    from tiny_inference_server_amd.architectures.gqa_mtp import _block, _norm
    layers = tuple(_block(cfg, f"transformer_block_list.{l}.") for l in range(3))
    calls = (LayerCall(0), LayerCall(1), LayerCall(2, cache="trunk.0", writes_cache=False), LayerCall(1))
    stage = StageSpec("trunk", 0, PartSpec("stage_input", "token_embedding"), calls, _norm(cfg, "rms_out.scale"))
    return ModelSpec(cfg.d_model, cfg.vocab_size, cfg.max_context, layers, (stage,), "embedding.weight", "embedding.weight")


def run_order_plain(ids, w, cfg, shared=True):
    """Blocks 0, 1, 2, 1 in that order; block 2 makes queries of its own and attends to block 0's keys and values
    (shared=False: to its own, as an ordinary block would)."""
    T, D, NH, G = len(ids), cfg.d_model, cfg.n_heads, cfg.group_size
    hd, pos = D // NH, torch.arange(T)
    pcfg = {"n_heads": NH, "group": G, "eps": cfg.rms_eps, "base": cfg.rope_base}
    x = w["embedding.weight"][torch.tensor(ids)]
    pre = "transformer_block_list.0."
    a = pm.rms_norm(x, w[pre + "att.rms_norm_att.scale"], cfg.rms_eps)
    k0, v0 = (a @ w[pre + "att.kv_proj.weight"]).view(T, 2, NH // G, hd).unbind(1)
    k0 = pm.apply_rope(k0, pos, cfg.rope_base)
    x = pm.block(x, w, pre, pcfg, pos)
    x = pm.block(x, w, "transformer_block_list.1.", pcfg, pos)
    pre = "transformer_block_list.2."
    a = pm.rms_norm(x, w[pre + "att.rms_norm_att.scale"], cfg.rms_eps)
    q = pm.apply_rope((a @ w[pre + "att.q_proj.weight"]).view(T, NH, hd), pos, cfg.rope_base)
    if not shared:
        k0, v0 = (a @ w[pre + "att.kv_proj.weight"]).view(T, 2, NH // G, hd).unbind(1)
        k0 = pm.apply_rope(k0, pos, cfg.rope_base)
    x = x + pm.causal_gqa_attention(q, k0, v0, G).reshape(T, D) @ w[pre + "att.linear_proj.weight"]
    f = pm.rms_norm(x, w[pre + "rms_norm_ffn.scale"], cfg.rms_eps)
    x = x + pm.swiglu_ffn(f, w[pre + "ffn.swig.linear1.weight"], w[pre + "ffn.swig.linear2.weight"], w[pre + "ffn.fc.weight"])
    x = pm.block(x, w, "transformer_block_list.1.", pcfg, pos)
    return pm.rms_norm(x, w["rms_out.scale"], cfg.rms_eps) @ w["embedding.weight"].T


@pytest.mark.parametrize("backend", [pytest.param("hip", marks=pytest.mark.gpu), "torch"])
@pytest.mark.parametrize("dtype,tol", [("float32", 2e-5), ("bfloat16", 2e-2)])
def test_a_layer_runs_twice_and_a_layer_reads_another_layers_cache(dtype, tol, backend):
    """Four calls over three layers: layer 1 runs twice, each time with keys and values of its own, and layer 2 writes
    none: its queries meet what layer 0 wrote. Three caches for four calls; logits equal the plain model's under
    whole prompts, portions beside decoded tokens and portions of changing size, pages used again in between."""
    from tiny_inference_server_amd.config import ARCHITECTURES, Architecture
    from tiny_inference_server_amd.engine import Engine
    cfg = GqaMtpConfig(d_model=96, vocab_size=157, max_context=256, rope_base=1e4, n_heads=6, n_layers=3, ffn_hidden=72,
                       group_size=3, mtp_heads=0, architecture="RunOrderToy")
    ARCHITECTURES.register("RunOrderToy", Architecture("RunOrderToy", GqaMtpConfig, run_order_spec), replace=True)
    w = random_tensors(cfg, 33, std=0.1, gain_jitter=0.1, dtype=dtype)
    ops = TorchOps(dtype=torch.float32 if dtype == "float32" else torch.bfloat16) if backend == "torch" else None
    eng = Engine(config=cfg, tensors=w, dtype=dtype, page_size=16, max_tokens=192, max_requests=3, ops=ops)
    assert sorted(eng.model.cache_needs()) == ["trunk.0", "trunk.1", "trunk.3"]
    w64 = {k: v.double() for k, v in w.items()}
    reqs = {"a": H.random_ids(157, 70, 8), "b": H.random_ids(157, 45, 9), "c": H.random_ids(157, 52, 10)}
    want = {rid: run_order_plain(ids, w64, cfg) for rid, ids in reqs.items()}
    scale = max(1.0, max(v.abs().max().item() for v in want.values()))
    # whose keys and values layer 2 sees must matter, or this test could not fail: with its own the logits move
    assert (run_order_plain(reqs["b"], w64, cfg, shared=False) - want["b"]).abs().max().item() > 20 * tol * scale
    for trace in (H.whole_trace(reqs), H.mixed_trace(reqs, 3, 11)[0], H.portions_trace({"a": reqs["a"], "c": reqs["c"]}, 4),
                  H.tail_decode_trace(reqs, 20)):
        got, _ = H.run_trace(eng, trace, heads=False)
        assert got
        for (rid, p), lg in got.items():
            assert (lg.double() - want[rid][p]).abs().max().item() <= tol * scale, (rid, p)
        eng.cache.check()
        assert eng.free_pages() == eng.total_pages()
    ARCHITECTURES.unregister("RunOrderToy")

"""How a model is put together from a spec, on the host: named parts of a block, cache keys for blocks with several
mixers, host planning found through the parts, graph promises. The kernels' stand-in runs the steps."""
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

            def plan_attention(self, n_heads, n_kv_heads, head_dim, seq_rows, add, mode=None):
                self.asked.append((n_heads, n_kv_heads, head_dim))
                return {("toy", n_heads): (add([1, 2, 3]), len(seq_rows))}

        ops = Planning()
        model = Model(spec, w, ops)
        got = model.plan_rows([(0, 0, 3), (3, 5, 1)], lambda a: 7)
        assert ops.asked == [(4, 2, 12)] and got == {("toy", 4): (7, 2)}      # three calls of two layers, one shape
    finally:
        MIXERS.unregister("_recurrence")
        ARRANGEMENTS.unregister("_both")

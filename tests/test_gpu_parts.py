"""Each part alone on the GPU against the plain implementation's function for it, and a toy mixer with state of
its own that is registered, built and stepped from here without touching the framework's files."""
import math
from dataclasses import dataclass

import pytest
import torch

import helpers as H
import plain_model as pm
from tiny_inference_server_amd.cache import CacheManager
from tiny_inference_server_amd.config import ARCHITECTURES, Architecture
from tiny_inference_server_amd.engine import Engine
from tiny_inference_server_amd.engine.batch import Entry, build_step_batch
from tiny_inference_server_amd.parts import (ARRANGEMENTS, MIXERS, POSITION_ENCODINGS, CallContext, LayerCall, LayerSpec, ModelSpec, PartSpec,
                                             StageSpec, StateNeed, Tensors, build_part, to_compute)
from tiny_inference_server_amd.weights import random_tensors

pytestmark = pytest.mark.gpu

DT = [("float32", torch.float32, 2e-5), ("bfloat16", torch.bfloat16, 3e-2)]


def ops_of(dtype):
    from tiny_inference_server_amd.ops.hip_ops import HipOps
    return HipOps("cuda:0", dtype)


def rnd(shape, seed, scale=1.0):
    return scale * torch.randn(shape, generator=torch.Generator().manual_seed(seed))


@pytest.mark.parametrize("name,dtype,tol", DT)
def test_norm_part(name, dtype, tol):
    ops = ops_of(dtype)
    gain = (1 + 0.1 * rnd((200,), 1)).to(dtype)
    part = build_part(PartSpec("norm", "rmsnorm_l2", {"width": 200, "eps": 1e-5}, {"gain": "g"}), Tensors({"g": gain}), ops)
    x = rnd((7, 200), 2, 3.0).to(dtype)
    want = pm.rms_norm(x.double(), gain.double(), 1e-5)
    assert (part(x.cuda()).cpu().double() - want).abs().max() <= tol * want.abs().max()


def test_rotary_part_table():
    ops = ops_of(torch.float32)
    part = build_part(PartSpec("position", "rotary", {"head_dim": 48, "base": 5e5, "max_context": 300, "pairing": "half"}),
                      Tensors({}), ops)
    table, interleaved = part.rotary()
    cos, sin = pm.rope_tables(300, 48, 5e5)
    assert not interleaved and table.shape == (300, 24, 2)
    torch.testing.assert_close(table[..., 0].cpu().double(), cos[:, :24], atol=2e-5, rtol=0)      # angles up to 300 in 32-bit
    torch.testing.assert_close(table[..., 1].cpu().double(), sin[:, :24], atol=2e-5, rtol=0)
    with pytest.raises(ValueError, match="pairing"):
        build_part(PartSpec("position", "rotary", {"head_dim": 8, "base": 1e4, "max_context": 8, "pairing": "odd"}), Tensors({}), ops)


@pytest.mark.parametrize("name,dtype,tol", DT)
def test_feed_forward_part(name, dtype, tol):
    ops = ops_of(dtype)
    D, Fh = 96, 200
    t = {"g": rnd((D, Fh), 3, D ** -0.5).to(dtype), "u": rnd((D, Fh), 4, D ** -0.5).to(dtype), "d": rnd((Fh, D), 5, Fh ** -0.5).to(dtype)}
    part = build_part(PartSpec("feed_forward", "swiglu", {"d_model": D, "hidden": Fh}, {"gate": "g", "up": "u", "down": "d"}),
                      Tensors(t), ops)
    x, res = rnd((9, D), 6).to(dtype), rnd((9, D), 7).to(dtype)
    want = res.double() + pm.swiglu_ffn(x.double(), t["g"].double(), t["u"].double(), t["d"].double())
    got = part.forward(x.cuda(), residual=res.cuda()).cpu().double()
    assert (got - want).abs().max() <= tol * want.abs().max()


def one_sequence_batch(needs, n_rows, page_size, dtype, start=0):
    cache = CacheManager(needs, page_size, 16, 2, dtype, torch.device("cuda:0"))
    slot = cache.open_request()
    cache.grow(slot, start + n_rows)
    step = build_step_batch([Entry(slot, start, list(range(n_rows)), [])], [0], [False], cache, torch.device("cuda:0"), 4096)
    return cache, step.stages[0]


@pytest.mark.parametrize("name,dtype,tol", DT)
@pytest.mark.parametrize("n_heads,n_kv,hd", [(4, 2, 16), (3, 1, 32), (6, 2, 8)])
def test_attention_mixer_and_block(name, dtype, tol, n_heads, n_kv, hd):
    ops = ops_of(dtype)
    D, Fh, T, eps, base = n_heads * hd, 72, 21, 1e-6, 1000.0
    pos = PartSpec("position", "rotary", {"head_dim": hd, "base": base, "max_context": 64, "pairing": "half"})
    mixer = PartSpec("mixer", "gqa_attention", {"d_model": D, "n_heads": n_heads, "n_kv_heads": n_kv, "head_dim": hd,
                                                "window": 0, "position": pos},
                     {"q": "b.att.q_proj.weight", "kv": "b.att.kv_proj.weight", "o": "b.att.linear_proj.weight"})
    norm = lambda n: PartSpec("norm", "rmsnorm_l2", {"width": D, "eps": eps}, {"gain": n})
    ffn = PartSpec("feed_forward", "swiglu", {"d_model": D, "hidden": Fh},
                   {"gate": "b.ffn.swig.linear1.weight", "up": "b.ffn.swig.linear2.weight", "down": "b.ffn.fc.weight"})
    layer = LayerSpec("prenorm_residual", {"mixer": mixer, "mixer_norm": norm("b.att.rms_norm_att.scale"),
                                           "feed_forward": ffn, "feed_forward_norm": norm("b.rms_norm_ffn.scale")})
    t = {"b.att.q_proj.weight": rnd((D, D), 10, D ** -0.5), "b.att.kv_proj.weight": rnd((D, 2 * n_kv * hd), 11, D ** -0.5),
         "b.att.linear_proj.weight": rnd((D, D), 12, D ** -0.5), "b.ffn.swig.linear1.weight": rnd((D, Fh), 13, D ** -0.5),
         "b.ffn.swig.linear2.weight": rnd((D, Fh), 14, D ** -0.5), "b.ffn.fc.weight": rnd((Fh, D), 15, Fh ** -0.5),
         "b.att.rms_norm_att.scale": 1 + 0.1 * rnd((D,), 16), "b.rms_norm_ffn.scale": 1 + 0.1 * rnd((D,), 17)}
    t = {k: v.to(dtype) for k, v in t.items()}
    block = ARRANGEMENTS.get("prenorm_residual")(layer, Tensors(t), ops)
    need = block.mixer.cache_need(mixer.params)
    cache, b = one_sequence_batch({"k": need}, T, 16, dtype)
    group = cache.group_of["k"]
    ctx = CallContext(batch=b, group=group, plane=cache.groups[group].plane("k"))
    x = rnd((T, D), 18).to(dtype)
    cfg = {"n_heads": n_heads, "group": n_heads // n_kv, "eps": eps, "base": base}
    w64 = {k: v.double() for k, v in t.items()}
    want = pm.block(x.double(), w64, "b.", cfg, torch.arange(T))
    got = block.forward(x.cuda(), ctx).cpu().double()
    assert (got - want).abs().max() <= tol * want.abs().max()
    # the mixer alone: out = attention(norm'd input) . Wo + residual
    a = pm.rms_norm(x.double(), w64["b.att.rms_norm_att.scale"], eps)
    q = pm.apply_rope((a @ w64["b.att.q_proj.weight"]).view(T, n_heads, hd), torch.arange(T), base)
    kv = (a @ w64["b.att.kv_proj.weight"]).view(T, 2, n_kv, hd)
    k = pm.apply_rope(kv[:, 0], torch.arange(T), base)
    o = pm.causal_gqa_attention(q, k, kv[:, 1], n_heads // n_kv).reshape(T, D) @ w64["b.att.linear_proj.weight"]
    got = block.mixer.forward(a.to(dtype).cuda(), ctx).cpu().double()
    assert (got - o).abs().max() <= tol * max(1.0, o.abs().max())


# ---- a toy mixer with state of its own, and a toy architecture around it: defined in tests/toy_parts.py ------------

from toy_parts import ToyConfig, ToyDecayMixer, toy_plain, toy_spec


def test_toy_mixer_with_state_is_registered_built_and_stepped():
    ARCHITECTURES.register("ToyStateModel", Architecture("ToyStateModel", ToyConfig, toy_spec), replace=True)
    MIXERS.register("toy_decay", ToyDecayMixer, replace=True)
    cfg = ToyConfig(d_model=48, vocab_size=101, hidden=80, decay=0.7)
    w = random_tensors(cfg, 9, std=0.1, gain_jitter=0.1, dtype="float32")
    eng = Engine(config=cfg, tensors=w, dtype="float32", page_size=16, max_tokens=64, max_requests=3)
    assert sorted(eng.model.cache_needs()) == ["trunk.0", "trunk.1", "trunk.2"] and not eng.cache.groups
    reqs = {"a": H.random_ids(101, 23, 1), "b": H.random_ids(101, 9, 2)}
    main = {}
    # whole, then in portions beside each other, then a slot used again by a new request
    for trace in (H.whole_trace(reqs), H.mixed_trace(reqs, 2, 3)[0], H.portions_trace({"b": reqs["b"]}, 1)):
        got, _ = H.run_trace(eng, trace, heads=False)
        for (rid, p), lg in got.items():
            want = toy_plain(reqs[rid], w, cfg)[p]
            assert (lg.double() - want).abs().max() <= 2e-5 * max(1.0, want.abs().max()), (rid, p)
    # the mixer promises graph safety for steps of single tokens only: those are captured and replayed, with the
    # state living in the request's slot between replays, and portions run as plain launches
    assert eng.use_decode_graphs and not eng.use_graphs
    replays = eng.graph_replays
    got, _ = H.run_trace(eng, H.tail_decode_trace(reqs, 8), heads=False)
    assert eng.graph_replays >= replays + 5
    for (rid, p), lg in got.items():
        want = toy_plain(reqs[rid], w, cfg)[p]
        assert (lg.double() - want).abs().max() <= 2e-5 * max(1.0, want.abs().max()), (rid, p)
    ARCHITECTURES.unregister("ToyStateModel")
    MIXERS.unregister("toy_decay")


def test_command_line_and_generate_take_a_toy_architecture(tmp_path, capsys):
    """The command line and generate() with a model folder of an architecture registered from here, whose
    configuration class is not the built-in one and whose mixers keep no pages: the pool's size in bytes is turned
    into pages by what the parts keep (nothing), the prompts are drawn from the spec's vocabulary, and the tokens
    are the plain toy model's."""
    from tiny_inference_server_amd.__main__ import main
    from tiny_inference_server_amd.engine.generate import generate
    from tiny_inference_server_amd.weights import write_random_model
    ARCHITECTURES.register("ToyStateModel", Architecture("ToyStateModel", ToyConfig, toy_spec), replace=True)
    MIXERS.register("toy_decay", ToyDecayMixer, replace=True)
    try:
        cfg = ToyConfig(d_model=48, vocab_size=101, hidden=80, decay=0.7)
        folder = write_random_model(cfg, 9, str(tmp_path / "toy"), std=0.1, gain_jitter=0.1, dtype="float32")
        w = random_tensors(cfg, 9, std=0.1, gain_jitter=0.1, dtype="float32")

        def greedy(prompt, n):
            ids = list(prompt)
            for _ in range(n):
                ids.append(int(torch.argmax(toy_plain(ids, w, cfg)[-1])))
            return ids[len(prompt):]
        prompts = [H.random_ids(101, n, 60 + i) for i, n in enumerate((11, 3, 17))]
        assert generate(folder, prompts, max_new_tokens=5, temperature=0.0, dtype="float32", max_batch=2,
                        token_budget=8) == [greedy(p, 5) for p in prompts]
        capsys.readouterr()
        assert main(["--model", folder, "--dtype", "float32", "--prompt-ids", "5,17,3", "--prompt-ids", "9",
                     "--max-new-tokens", "4", "--greedy", "--pool-bytes", "1MiB", "--max-batch", "2"]) == 0
        lines = [l.split()[1:] for l in capsys.readouterr().out.splitlines() if l.startswith("OUTPUT:")]
        assert [[int(t) for t in l] for l in lines] == [greedy([5, 17, 3], 4), greedy([9], 4)]
    finally:
        ARCHITECTURES.unregister("ToyStateModel")
        MIXERS.unregister("toy_decay")


# ---- toy arrangements: a block with no feed-forward, and a block with two mixers, each with a cache of its own ------

def register_toy_arrangements():
    from tiny_inference_server_amd.parts import Arrangement

    @ARRANGEMENTS.register("toy_mixer_only", replace=True)
    class ToyMixerOnly(Arrangement):
        """x = x + mixer(norm(x)): no feed-forward at all."""
        part_names = ("norm", "mixer")

        def forward(self, x, ctx):
            return self.parts["mixer"].forward(self.parts["norm"](x), ctx.of("mixer"), residual=x)

    @ARRANGEMENTS.register("toy_two_mixers", replace=True)
    class ToyTwoMixers(Arrangement):
        """x = x + attention(norm(x)) + decay(norm(x)): two mixers read the same normed rows; one has pages, the other
        a state slot."""
        part_names = ("norm", "attention", "decay")

        def forward(self, x, ctx):
            a = self.parts["norm"](x)
            x = self.parts["attention"].forward(a, ctx.of("attention"), residual=x)
            return self.parts["decay"].forward(a, ctx.of("decay"), residual=x)


def toy_arrangement_spec(cfg):
    from tiny_inference_server_amd.architectures.gqa_mtp import _block, _norm
    layers = []
    for l in range(3):
        blk = _block(cfg, f"transformer_block_list.{l}.")
        norm, att = blk.part("mixer_norm"), blk.part("mixer")
        decay = PartSpec("mixer", "toy_decay", {"d_model": cfg.d_model, "decay": 0.6}, {"w": f"l{l}.decay.w"})
        if l == 0:
            layers.append(LayerSpec("toy_mixer_only", {"norm": norm, "mixer": att}))
        elif l == 1:
            layers.append(LayerSpec("toy_two_mixers", {"norm": norm, "attention": att, "decay": decay}))
        else:
            layers.append(blk)
    stage = StageSpec("trunk", 0, PartSpec("stage_input", "token_embedding"), tuple(LayerCall(l) for l in range(3)),
                      _norm(cfg, "rms_out.scale"))
    return ModelSpec(cfg.d_model, cfg.vocab_size, cfg.max_context, tuple(layers), (stage,), "embedding.weight", "embedding.weight")


def toy_arrangement_plain(ids, w, cfg):
    T, D, NH, G = len(ids), cfg.d_model, cfg.n_heads, cfg.group_size
    hd, pos = D // NH, torch.arange(len(ids))
    x = w["embedding.weight"][torch.tensor(ids)]

    def attention(a, pre):
        q = pm.apply_rope((a @ w[pre + "att.q_proj.weight"]).view(T, NH, hd), pos, cfg.rope_base)
        k, v = (a @ w[pre + "att.kv_proj.weight"]).view(T, 2, NH // G, hd).unbind(1)
        return pm.causal_gqa_attention(q, pm.apply_rope(k, pos, cfg.rope_base), v, G).reshape(T, D) @ w[pre + "att.linear_proj.weight"]

    for l in range(3):
        pre = f"transformer_block_list.{l}."
        a = pm.rms_norm(x, w[pre + "att.rms_norm_att.scale"], cfg.rms_eps)
        x = x + attention(a, pre)
        if l == 1:
            s, rows = torch.zeros(D, dtype=torch.float64), []
            for r in range(T):
                s = 0.6 * s + a[r]
                rows.append(s)
            x = x + torch.stack(rows) @ w["l1.decay.w"]
        if l == 2:
            f = pm.rms_norm(x, w[pre + "rms_norm_ffn.scale"], cfg.rms_eps)
            x = x + pm.swiglu_ffn(f, w[pre + "ffn.swig.linear1.weight"], w[pre + "ffn.swig.linear2.weight"], w[pre + "ffn.fc.weight"])
    return pm.rms_norm(x, w["rms_out.scale"], cfg.rms_eps) @ w["embedding.weight"].T


def test_toy_blocks_without_feed_forward_and_with_two_mixers():
    """Which parts a block has is the arrangement's business. From here, with no dummy parts and no change to the
    framework: a block of norm and attention alone, and a block whose two mixers (attention with pages, a recurrence
    with a state slot) each get a cache of their own; beside the built-in block. The loader asks for exactly the
    tensors these parts name."""
    from tiny_inference_server_amd.config import GqaMtpConfig
    from tiny_inference_server_amd.weights.loader import spec_tensors
    register_toy_arrangements()
    MIXERS.register("toy_decay", ToyDecayMixer, replace=True)
    cfg = GqaMtpConfig(d_model=80, vocab_size=131, max_context=256, rope_base=1e4, n_heads=5, n_layers=3, ffn_hidden=56,
                       group_size=5, mtp_heads=0, architecture="ToyArrangements")
    ARCHITECTURES.register("ToyArrangements", Architecture("ToyArrangements", GqaMtpConfig, toy_arrangement_spec), replace=True)
    names = set(spec_tensors(toy_arrangement_spec(cfg)))
    assert "l1.decay.w" in names and not any(n.startswith(("transformer_block_list.0.ffn", "transformer_block_list.1.ffn",
                                                            "transformer_block_list.0.rms_norm_ffn")) for n in names)
    w = {n: 0.1 * rnd(sh, 40 + i) if len(sh) > 1 else 1 + 0.1 * rnd(sh, 40 + i)
         for i, (n, sh) in enumerate(sorted(spec_tensors(toy_arrangement_spec(cfg)).items()))}
    eng = Engine(config=cfg, tensors=w, dtype="float32", page_size=16, max_tokens=256, max_requests=3)
    needs = eng.model.cache_needs()
    assert sorted(needs) == ["trunk.0", "trunk.1:attention", "trunk.1:decay", "trunk.2"]
    assert isinstance(needs["trunk.1:decay"], StateNeed) and len(eng.cache.groups) == 1
    w64 = {k: v.double() for k, v in w.items()}
    reqs = {"a": H.random_ids(131, 41, 5), "b": H.random_ids(131, 19, 6)}
    for trace in (H.whole_trace(reqs), H.mixed_trace(reqs, 2, 7)[0], H.portions_trace({"a": reqs["a"]}, 3)):
        got, _ = H.run_trace(eng, trace, heads=False)
        assert got
        for (rid, p), lg in got.items():
            want = toy_arrangement_plain(reqs[rid], w64, cfg)[p]
            assert (lg.double() - want).abs().max() <= 2e-5 * max(1.0, want.abs().max()), (rid, p)
    ARCHITECTURES.unregister("ToyArrangements")
    MIXERS.unregister("toy_decay")
    ARRANGEMENTS.unregister("toy_mixer_only")
    ARRANGEMENTS.unregister("toy_two_mixers")


# ---- layers with different cache needs in one model: a sliding window beside full attention ----------------------

def windowed_spec(cfg, windows):
    from tiny_inference_server_amd.architectures.gqa_mtp import _block, _norm
    import dataclasses
    layers = []
    for l, win in enumerate(windows):
        blk = _block(cfg, f"transformer_block_list.{l}.")
        mixer = blk.part("mixer")
        layers.append(blk.with_part("mixer", dataclasses.replace(mixer, params={**mixer.params, "window": win})))
    stage = StageSpec("trunk", 0, PartSpec("stage_input", "token_embedding"), tuple(LayerCall(l) for l in range(len(windows))),
                      _norm(cfg, "rms_out.scale"))
    return ModelSpec(cfg.d_model, cfg.vocab_size, cfg.max_context, tuple(layers), (stage,), "embedding.weight", "embedding.weight")


@pytest.mark.parametrize("dtype,tol", [("float32", 2e-5), ("bfloat16", 2e-2)])
def test_window_layers_get_pages_of_their_own_and_give_them_back(dtype, tol):
    """Layer 0 sees the last 24 keys, layer 1 all of them, layer 2 the last 40: three page groups. Window groups hold
    few pages however long the request grows, and the logits equal the plain model's with the same windows."""
    from tiny_inference_server_amd.config import GqaMtpConfig
    windows = (24, 0, 40)
    cfg = GqaMtpConfig(d_model=128, vocab_size=211, max_context=512, rope_base=1e4, n_heads=4, n_layers=3, ffn_hidden=160,
                       group_size=2, mtp_heads=0, architecture="WindowedToy")
    ARCHITECTURES.register("WindowedToy", Architecture("WindowedToy", GqaMtpConfig, lambda c: windowed_spec(c, windows)),
                           replace=True)
    w = random_tensors(cfg, 21, std=0.08, gain_jitter=0.1, dtype=dtype)
    eng = Engine(config=cfg, tensors=w, dtype=dtype, page_size=16, max_tokens=512, max_requests=2)
    assert len(eng.cache.groups) == 3
    ids = H.random_ids(211, 300, 5)
    # plain: the same blocks with their windows
    w64 = {k: v.double() for k, v in w.items()}
    pcfg = {"n_heads": 4, "group": 2, "eps": cfg.rms_eps, "base": 1e4}
    x = w64["embedding.weight"][torch.tensor(ids)]
    for l, win in enumerate(windows):
        x = pm.block(x, w64, f"transformer_block_list.{l}.", pcfg, torch.arange(len(ids)), window=win)
    want = pm.rms_norm(x, w64["rms_out.scale"], cfg.rms_eps) @ w64["embedding.weight"].T
    # a long portion, portions that end inside and on page edges, then token by token
    got, p = {}, 0
    for n in [100, 37, 27, 16, 1, 1, 30] + [1] * 88:
        out = eng.step([("a", ids[p:p + n], list(range(n)))])
        lg = out.logits.float().cpu()
        for i in range(n):
            got[p + i] = lg[i]
        p += n
        held = {name: g.held(eng.requests["a"][0]) for name, g in eng.cache.groups.items()}
        assert held["kv2x32"] == -(-p // 16)
        assert held["kv2x32w24"] <= 24 // 16 + 2 and held["kv2x32w40"] <= 40 // 16 + 2
    assert p == 300
    scale = max(1.0, want.abs().max().item())
    worst = max((got[i].double() - want[i]).abs().max().item() for i in range(300))
    assert worst <= tol * scale, worst
    eng.close("a")
    eng.cache.check()
    assert eng.cache.free_pages() == eng.cache.total_pages()
    ARCHITECTURES.unregister("WindowedToy")


# ---- a toy feed-forward with routing and a toy position encoding, defined here, in the built-in block ------------

from tiny_inference_server_amd.parts import FEED_FORWARDS, POSITION_ENCODINGS


class ToyTop1Experts:
    """Each row goes to the expert its router logit is largest for; y = p * expert(x), p being the softmax weight of
    the chosen expert. Router logits and their softmax are 32-bit. An expert is a dense gated feed-forward."""

    @classmethod
    def tensor_shapes(cls, params):
        d, f, e = params["d_model"], params["hidden"], params["n_experts"]
        shapes = {"router": (d, e)}
        for i in range(e):
            shapes.update({f"gate{i}": (d, f), f"up{i}": (d, f), f"down{i}": (f, d)})
        return shapes

    def __init__(self, spec, tensors, ops):
        self.ops, self.n = ops, int(spec.params["n_experts"])
        self.router = to_compute(ops, tensors.of(spec, "router").t())
        self.gate_up, self.down = [], []
        for i in range(self.n):
            g, u = tensors.of(spec, f"gate{i}"), tensors.of(spec, f"up{i}")
            self.gate_up.append(to_compute(ops, torch.stack((g.t(), u.t()), dim=1).reshape(2 * g.shape[1], g.shape[0])))
            self.down.append(to_compute(ops, tensors.of(spec, f"down{i}").t()))

    def forward(self, x, residual=None):
        logits = self.ops.linear(x, self.router, out_dtype=torch.float32)
        prob, choice = torch.softmax(logits, dim=-1).max(dim=-1)
        out = residual.clone() if residual is not None else torch.zeros_like(x)
        for e in range(self.n):
            rows = (choice == e).nonzero().flatten()
            if rows.numel():
                y = self.ops.linear(self.ops.linear_swiglu(x[rows].contiguous(), self.gate_up[e]), self.down[e])
                out[rows] = (out[rows].float() + prob[rows, None] * y.float()).to(out.dtype)
        return out


class ToyStretchedRotary:
    """Rotary encoding whose angle at position p is that of position p / stretch: another table, same kernels."""

    @classmethod
    def tensor_shapes(cls, params):
        return {}

    def __init__(self, spec, tensors, ops):
        p = spec.params
        hd, self.max_context = int(p["head_dim"]), int(p["max_context"])
        theta = 1.0 / torch.pow(torch.tensor(float(p["base"])), (2 * torch.arange(hd // 2).float()) / hd)
        angle = torch.outer(torch.arange(self.max_context).float() / float(p["stretch"]), theta)
        self.table = torch.stack((torch.cos(angle), torch.sin(angle)), dim=-1).contiguous().to(ops.device)

    def rotary(self):
        return self.table, False


def routed_spec(cfg, n_experts, stretch):
    from tiny_inference_server_amd.architectures.gqa_mtp import _block, _norm
    import dataclasses
    layers = []
    for l in range(cfg.n_layers):
        blk = _block(cfg, f"transformer_block_list.{l}.")
        pos = PartSpec("position", "toy_stretched_rotary", {"head_dim": cfg.head_dim, "base": cfg.rope_base,
                                                            "max_context": cfg.max_context, "stretch": stretch})
        mixer = dataclasses.replace(blk.part("mixer"), params={**blk.part("mixer").params, "position": pos})
        names = {"router": f"l{l}.router"}
        for e in range(n_experts):
            names.update({f"gate{e}": f"l{l}.e{e}.g", f"up{e}": f"l{l}.e{e}.u", f"down{e}": f"l{l}.e{e}.d"})
        ffn = PartSpec("feed_forward", "toy_top1_experts",
                       {"d_model": cfg.d_model, "hidden": cfg.ffn_hidden, "n_experts": n_experts}, names)
        # the second layer keeps the built-in dense feed-forward: parts are chosen layer by layer
        blk = blk.with_part("mixer", mixer)
        layers.append(blk.with_part("feed_forward", ffn) if l != 1 else blk)
    stage = StageSpec("trunk", 0, PartSpec("stage_input", "token_embedding"), tuple(LayerCall(l) for l in range(cfg.n_layers)),
                      _norm(cfg, "rms_out.scale"))
    return ModelSpec(cfg.d_model, cfg.vocab_size, cfg.max_context, tuple(layers), (stage,), "embedding.weight", "embedding.weight")


def routed_plain(ids, w, cfg, n_experts, stretch):
    T, D, NH, G = len(ids), cfg.d_model, cfg.n_heads, cfg.group_size
    KVH, hd = NH // G, D // NH
    x = w["embedding.weight"][torch.tensor(ids)]
    j = torch.arange(hd // 2, dtype=torch.float64)
    angle = torch.outer(torch.arange(T, dtype=torch.float64) / stretch, cfg.rope_base ** (-2 * j / hd))
    cos, sin = torch.cos(angle).repeat(1, 2).unsqueeze(1), torch.sin(angle).repeat(1, 2).unsqueeze(1)
    rope = lambda t: t * cos + pm.rotate_half(t) * sin
    for l in range(cfg.n_layers):
        pre = f"transformer_block_list.{l}."
        a = pm.rms_norm(x, w[pre + "att.rms_norm_att.scale"], cfg.rms_eps)
        q = (a @ w[pre + "att.q_proj.weight"]).view(T, NH, hd)
        k, v = (a @ w[pre + "att.kv_proj.weight"]).view(T, 2, KVH, hd).unbind(1)
        x = x + pm.causal_gqa_attention(rope(q), rope(k), v, G).reshape(T, D) @ w[pre + "att.linear_proj.weight"]
        f = pm.rms_norm(x, w[pre + "rms_norm_ffn.scale"], cfg.rms_eps)
        if l == 1:
            x = x + pm.swiglu_ffn(f, w[pre + "ffn.swig.linear1.weight"], w[pre + "ffn.swig.linear2.weight"], w[pre + "ffn.fc.weight"])
            continue
        prob, choice = torch.softmax(f @ w[f"l{l}.router"], dim=-1).max(dim=-1)
        y = torch.stack([pm.swiglu_ffn(f[r], w[f"l{l}.e{int(choice[r])}.g"], w[f"l{l}.e{int(choice[r])}.u"],
                                        w[f"l{l}.e{int(choice[r])}.d"]) for r in range(T)])
        x = x + prob[:, None] * y
    return pm.rms_norm(x, w["rms_out.scale"], cfg.rms_eps) @ w["embedding.weight"].T


class ToyDistanceBias:
    """A position encoding that leaves queries and keys alone and lowers a score by slope[h] per position of distance."""

    @classmethod
    def tensor_shapes(cls, params):
        return {}

    def __init__(self, spec, tensors, ops):
        self.ops, self.steepest = ops, float(spec.params["steepest"])
        self.max_context = int(spec.params["max_context"])

    def rotary(self):
        return None, False

    def score_slopes(self, n_heads):
        return (self.steepest * 2.0 ** -torch.arange(n_heads, dtype=torch.float32)).to(self.ops.device)


def distance_bias_spec(cfg, steepest):
    from tiny_inference_server_amd.architectures.gqa_mtp import _block, _norm
    import dataclasses
    layers = []
    for l in range(cfg.n_layers):
        blk = _block(cfg, f"transformer_block_list.{l}.")
        pos = PartSpec("position", "toy_distance_bias", {"steepest": steepest, "max_context": cfg.max_context})
        layers.append(blk.with_part("mixer", dataclasses.replace(blk.part("mixer"),
                                                                 params={**blk.part("mixer").params, "position": pos})))
    stage = StageSpec("trunk", 0, PartSpec("stage_input", "token_embedding"), tuple(LayerCall(l) for l in range(cfg.n_layers)),
                      _norm(cfg, "rms_out.scale"))
    return ModelSpec(cfg.d_model, cfg.vocab_size, cfg.max_context, tuple(layers), (stage,), "embedding.weight", "embedding.weight")


def distance_bias_plain(ids, w, cfg, steepest):
    T, D, NH, G = len(ids), cfg.d_model, cfg.n_heads, cfg.group_size
    KVH, hd = NH // G, D // NH
    x = w["embedding.weight"][torch.tensor(ids)]
    dist = (torch.arange(T)[None, :] - torch.arange(T)[:, None]).double()          # key position - row position
    causal = dist <= 0
    for l in range(cfg.n_layers):
        pre = f"transformer_block_list.{l}."
        a = pm.rms_norm(x, w[pre + "att.rms_norm_att.scale"], cfg.rms_eps)
        q = (a @ w[pre + "att.q_proj.weight"]).view(T, NH, hd)
        k, v = (a @ w[pre + "att.kv_proj.weight"]).view(T, 2, KVH, hd).unbind(1)
        heads = []
        for h in range(NH):
            s = (q[:, h] @ k[:, h // G].T) * hd ** -0.5 + steepest * 2.0 ** -h * dist
            heads.append(torch.softmax(s.masked_fill(~causal, float("-inf")), dim=-1) @ v[:, h // G])
        x = x + torch.stack(heads, dim=1).reshape(T, D) @ w[pre + "att.linear_proj.weight"]
        f = pm.rms_norm(x, w[pre + "rms_norm_ffn.scale"], cfg.rms_eps)
        x = x + pm.swiglu_ffn(f, w[pre + "ffn.swig.linear1.weight"], w[pre + "ffn.swig.linear2.weight"], w[pre + "ffn.fc.weight"])
    return pm.rms_norm(x, w["rms_out.scale"], cfg.rms_eps) @ w["embedding.weight"].T


@pytest.mark.parametrize("dtype,tol", [("float32", 2e-5), ("bfloat16", 3e-2)])
def test_toy_position_encoding_that_works_on_the_scores(dtype, tol):
    """Not every position encoding rotates: one that adds a bias to the scores, linear in the distance and with a
    slope per head, is registered from here and runs inside the framework's attention mixer (the general kernel takes
    such calls). Without the bias the logits would differ by far more than the tolerance (checked)."""
    from tiny_inference_server_amd.config import GqaMtpConfig
    POSITION_ENCODINGS.register("toy_distance_bias", ToyDistanceBias, replace=True)
    steepest = 0.5
    cfg = GqaMtpConfig(d_model=96, vocab_size=149, max_context=256, rope_base=1e4, n_heads=6, n_layers=2, ffn_hidden=80,
                       group_size=2, mtp_heads=0, architecture="DistanceBiasToy")
    ARCHITECTURES.register("DistanceBiasToy", Architecture("DistanceBiasToy", GqaMtpConfig,
                                                           lambda c: distance_bias_spec(c, steepest)), replace=True)
    w = random_tensors(cfg, 37, std=0.1, gain_jitter=0.1, dtype="float32")
    if dtype == "bfloat16":
        w = {k: v.to(torch.bfloat16) for k, v in w.items()}
    w64 = {k: v.double() for k, v in w.items()}
    eng = Engine(config=cfg, tensors=w, dtype=dtype, page_size=16, max_tokens=256, max_requests=3)
    reqs = {"a": H.random_ids(149, 52, 8), "b": H.random_ids(149, 21, 9)}
    want = {rid: distance_bias_plain(ids, w64, cfg, steepest) for rid, ids in reqs.items()}
    flat = {rid: distance_bias_plain(ids, w64, cfg, 0.0) for rid, ids in reqs.items()}
    scale = max(t.abs().max().item() for t in want.values())
    assert max((want[r] - flat[r]).abs().max().item() for r in reqs) > 20 * tol * scale
    for trace in (H.whole_trace(reqs), H.mixed_trace(reqs, 2, 5)[0], H.portions_trace({"a": reqs["a"]}, 7)):
        got, _ = H.run_trace(eng, trace, heads=False)
        assert got
        for (rid, p), lg in got.items():
            assert (lg.double() - want[rid][p]).abs().max() <= tol * max(1.0, scale), (rid, p)
    ARCHITECTURES.unregister("DistanceBiasToy")
    POSITION_ENCODINGS.unregister("toy_distance_bias")


def test_toy_routed_feed_forward_and_toy_position_encoding_in_the_built_in_block():
    """A feed-forward that routes rows to experts and a position encoding with another table are registered from
    here and used inside the framework's own block and attention mixer, layer by layer beside the built-in dense
    feed-forward; whole prompts, portions and mixed steps give the plain model's logits."""
    from tiny_inference_server_amd.config import GqaMtpConfig
    FEED_FORWARDS.register("toy_top1_experts", ToyTop1Experts, replace=True)
    POSITION_ENCODINGS.register("toy_stretched_rotary", ToyStretchedRotary, replace=True)
    n_experts, stretch = 3, 2.5
    cfg = GqaMtpConfig(d_model=96, vocab_size=157, max_context=256, rope_base=1e4, n_heads=6, n_layers=3, ffn_hidden=72,
                       group_size=3, mtp_heads=0, architecture="RoutedToy")
    ARCHITECTURES.register("RoutedToy", Architecture("RoutedToy", GqaMtpConfig, lambda c: routed_spec(c, n_experts, stretch)),
                           replace=True)
    w = random_tensors(cfg, 31, std=0.1, gain_jitter=0.1, dtype="float32")
    eng = Engine(config=cfg, tensors=w, dtype="float32", page_size=16, max_tokens=256, max_requests=3)
    assert not eng.use_graphs and not eng.use_decode_graphs      # the routed part made no promise about graph capture
    w64 = {k: v.double() for k, v in w.items()}
    reqs = {"a": H.random_ids(157, 45, 3), "b": H.random_ids(157, 18, 4)}
    used = set()
    for trace in (H.whole_trace(reqs), H.mixed_trace(reqs, 2, 5)[0], H.portions_trace({"a": reqs["a"]}, 7)):
        got, _ = H.run_trace(eng, trace, heads=False)
        for (rid, p), lg in got.items():
            want = routed_plain(reqs[rid], w64, cfg, n_experts, stretch)[p]
            assert (lg.double() - want).abs().max() <= 2e-5 * max(1.0, want.abs().max()), (rid, p)
    for l in (0, 2):          # the routing is not trivial: more than one expert is chosen in a prompt
        f = pm.rms_norm(w64["embedding.weight"][torch.tensor(reqs["a"])], w64[f"transformer_block_list.{l}.rms_norm_ffn.scale"], cfg.rms_eps)
        used.add(len(set((f @ w64[f"l{l}.router"]).argmax(-1).tolist())))
    assert max(used) > 1
    ARCHITECTURES.unregister("RoutedToy")
    FEED_FORWARDS.unregister("toy_top1_experts")
    POSITION_ENCODINGS.unregister("toy_stretched_rotary")

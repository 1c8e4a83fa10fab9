"""A toy mixer with state of its own and a toy architecture around it, defined in the tests and registered from there:
nothing under tiny_inference_server_amd/ knows of them."""
from dataclasses import dataclass

import torch

import plain_model as pm
from tiny_inference_server_amd.parts import (MIXERS, LayerCall, LayerSpec, ModelSpec, PartSpec, StageSpec, StateNeed,
                                             to_compute)

@MIXERS.register("toy_decay", replace=True)
class ToyDecayMixer:
    """s <- decay * s + x for every row in order; y = s . W (+ residual). Its state is one vector per request."""

    @classmethod
    def tensor_shapes(cls, params):
        return {"w": (params["d_model"], params["d_model"])}

    @classmethod
    def cache_need(cls, params):
        return StateNeed((params["d_model"],), "float32")

    def __init__(self, spec, tensors, ops):
        self.ops, self.decay = ops, float(spec.params["decay"])
        self.w = to_compute(ops, tensors.of(spec, "w").t())

    # a portion's rows are walked on the host; when every request brings one token the state is updated with the step's
    # device arrays alone, and such steps may be captured as graphs
    graph_safe = "single_rows"

    def forward(self, x, ctx, residual=None):
        b = ctx.batch
        if b.max_seq_rows == 1 and b.n_rows == b.n_seqs:
            slots = b.seq_slots.long()
            s = self.decay * ctx.state[slots] + x.float()
            ctx.state[slots] = s
            return self.ops.linear(s.to(x.dtype), self.w, residual=residual)
        s_all = torch.empty(x.shape[0], x.shape[1], dtype=torch.float32, device=x.device)
        for (first, p0, n), slot in zip(ctx.batch.seq_rows, ctx.batch.host_slots):
            s = ctx.state[slot]
            for r in range(first, first + n):
                s = self.decay * s + x[r].float()
                s_all[r] = s
            if n:
                ctx.state[slot] = s
        return self.ops.linear(s_all.to(x.dtype), self.w, residual=residual)


@dataclass(frozen=True)
class ToyConfig:
    d_model: int
    vocab_size: int
    hidden: int
    decay: float
    max_context: int = 128
    architecture: str = "ToyStateModel"

    @classmethod
    def from_dict(cls, raw):
        return cls(raw["d_model"], raw["vocab_size"], raw["hidden"], raw["decay"], raw.get("max_context", 128))

    def to_dict(self):
        return dict(self.__dict__)


def toy_spec(cfg):
    norm = lambda n: PartSpec("norm", "rmsnorm_l2", {"width": cfg.d_model, "eps": 1e-6}, {"gain": n})
    layers = []
    for l in range(2):
        mixer = PartSpec("mixer", "toy_decay", {"d_model": cfg.d_model, "decay": cfg.decay}, {"w": f"l{l}.mix.w"})
        ffn = PartSpec("feed_forward", "swiglu", {"d_model": cfg.d_model, "hidden": cfg.hidden},
                       {"gate": f"l{l}.g", "up": f"l{l}.u", "down": f"l{l}.d"})
        layers.append(LayerSpec("prenorm_residual", {"mixer": mixer, "mixer_norm": norm(f"l{l}.n1"),
                                                     "feed_forward": ffn, "feed_forward_norm": norm(f"l{l}.n2")}))
    # the run order is data: layer 0, layer 1, then layer 0 again with a state of its own
    stage = StageSpec("trunk", 0, PartSpec("stage_input", "token_embedding"),
                      (LayerCall(0), LayerCall(1), LayerCall(0)), norm("out"))
    return ModelSpec(cfg.d_model, cfg.vocab_size, cfg.max_context, tuple(layers), (stage,), "emb", "emb")


def toy_plain(ids, w, cfg):
    x = w["emb"][torch.tensor(ids)].double()
    for l in (0, 1, 0):
        a = pm.rms_norm(x, w[f"l{l}.n1"].double(), 1e-6)
        s, rows = torch.zeros(cfg.d_model, dtype=torch.float64), []
        for r in range(len(ids)):
            s = cfg.decay * s + a[r]
            rows.append(s)
        x = x + torch.stack(rows) @ w[f"l{l}.mix.w"].double()
        x = x + pm.swiglu_ffn(pm.rms_norm(x, w[f"l{l}.n2"].double(), 1e-6), w[f"l{l}.g"].double(), w[f"l{l}.u"].double(),
                              w[f"l{l}.d"].double())
    return pm.rms_norm(x, w["out"].double(), 1e-6) @ w["emb"].double().T



"""Attention mixers."""
from __future__ import annotations

import torch

from .base import MIXERS, build_part, to_compute
from .spec import PagedKvNeed


@MIXERS.register("gqa_attention")
class GqaAttention:
    """Grouped-query attention over a paged cache.

    q = x.Wq, [k|v] = x.Wkv, rotary on q and k, keys and values written into the call's cache plane before
    any row attends, then every row at position p attends the keys [0, p] (or the last `window`) of its
    own request, query head h using key/value head h // group_size; out = attn.Wo (+ residual)
    (reference main_models_new.py:96-136; paged_attention_kernels.py:49).

    params: d_model, n_heads, n_kv_heads, head_dim, window (0: all keys), position (a PartSpec).
    tensors: q (d_model, n_heads*head_dim), kv (d_model, 2*n_kv_heads*head_dim) with the key columns first,
    o (n_heads*head_dim, d_model); all stored [in, out] as the reference applies them (x @ W).
    """
    graph_safe = True

    @classmethod
    def tensor_shapes(cls, params):
        d, nh, nkv, hd = params["d_model"], params["n_heads"], params["n_kv_heads"], params["head_dim"]
        return {"q": (d, nh * hd), "kv": (d, 2 * nkv * hd), "o": (nh * hd, d)}

    @classmethod
    def cache_need(cls, params):
        return PagedKvNeed(params["n_kv_heads"], params["head_dim"], int(params.get("window", 0)))

    def __init__(self, spec, tensors, ops):
        p = spec.params
        self.ops = ops
        self.n_heads, self.n_kv_heads, self.head_dim = int(p["n_heads"]), int(p["n_kv_heads"]), int(p["head_dim"])
        if self.n_heads % self.n_kv_heads:
            raise ValueError(f"{self.n_heads} query heads are not a multiple of {self.n_kv_heads} key/value heads")
        self.window = int(p.get("window", 0))
        self.scale = float(p.get("scale", self.head_dim ** -0.5))
        pos = p["position"]
        self.position = build_part(pos, tensors, ops)
        # a position encoding may work on the scores instead of (or beside) rotating queries and keys
        slopes = getattr(self.position, "score_slopes", None)
        self.slopes = slopes(self.n_heads) if slopes is not None else None
        # one projection for q, k and v: rows of the [out, in] matrix are q heads, then k heads, then v heads.
        # Inside every q and k head the rows are put in pair order (the two members of a rotary pair side by side),
        # so that the kernel that makes them can rotate them while they are still in its registers.
        w = torch.cat((tensors.of(spec, "q"), tensors.of(spec, "kv")), dim=1).t()
        _, interleaved = self.position.rotary()
        hd, half = self.head_dim, self.head_dim // 2
        if not interleaved:
            order = torch.stack((torch.arange(half), torch.arange(half) + half), dim=1).reshape(-1)
            rows = torch.arange(w.shape[0]).view(-1, hd)
            n_qk = self.n_heads + self.n_kv_heads
            rows[:n_qk] = rows[:n_qk][:, order]
            w = w[rows.reshape(-1)]
        self.w_qkv = to_compute(ops, w)
        self.w_o = to_compute(ops, tensors.of(spec, "o").t())
        self.q_width = self.n_heads * self.head_dim

    fuses_norm = True

    # work lists for the attention kernels are made on the host, once per step and attention shape
    def plan_key(self):
        if not hasattr(self.ops, "plan_attention"):
            return None
        return ("attention", self.n_heads, self.n_kv_heads, self.head_dim, self.window)

    def plan_mode(self, seq_rows):
        mode = getattr(self.ops, "plan_attention_mode", None)
        return mode(seq_rows, self.window) if mode is not None else None

    def plan_rows(self, seq_rows, add, mode=None):
        return self.ops.plan_attention(self.n_heads, self.n_kv_heads, self.head_dim, seq_rows, add, mode, self.window)

    def forward(self, x, ctx, residual=None, norm=None):
        ops, b = self.ops, ctx.batch
        rms = None
        if norm is not None:
            if hasattr(norm, "as_rms"):
                rms = norm.as_rms()
            else:
                x = norm(x)
        table, interleaved = self.position.rotary()
        page_size = ctx.plane.shape[3]
        q = ops.qkv_rope(x, self.w_qkv, rms, b.positions, b.write_slots[ctx.group], table, ctx.plane, self.n_heads,
                         self.n_kv_heads, self.head_dim, page_size, interleaved, ctx.writes_cache)
        extra = {"slopes": self.slopes} if self.slopes is not None else {}
        attn = ops.paged_attention(q, ctx.plane, b, ctx.group, self.n_heads, self.n_kv_heads,
                                   self.head_dim, self.window, self.scale, **extra)
        return ops.linear(attn, self.w_o, residual=residual, reuse_residual=ctx.residual_is_spent)

"""A plain, slow implementation of the model, written from the reference's formulas.

Whole sequences, no cache, no batching, one function for each part, float64 by default. It shares no code
with the engine: it reads config.json and model.safetensors itself. Each function cites the lines of the
reference (main_models_new.py, server.py, ...) that it follows. The reference was read, not run.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional, Sequence

import torch


# ---- reading a model folder -----------------------------------------------------------------------------

def read_model_folder(model_dir: str, dtype=torch.float64):
    """(config dict with lower-case keys, {tensor name: tensor in `dtype`})."""
    from safetensors.torch import load_file
    with open(os.path.join(model_dir, "config.json")) as f:
        raw = json.load(f)
    cfg = {
        "d_model": raw["D_MODEL"], "vocab": raw["VOCAB_SIZE"], "max_context": raw["MAX_CONTEXT"],
        "base": float(raw["MAX_FREQ"]), "n_heads": raw["N_HEAD"], "n_layers": raw["NUM_LAYERS"],
        "ffn": raw["FFN_HIDDEN_DIM"], "group": raw["NUM_GROUPS"], "mtp": raw.get("MTP_HEADS", 0),
        "eps": float(raw.get("RMS_EPS", 2e-8)), "tied": bool(raw.get("TIE_EMBEDDINGS", True)),
    }
    weights = {k: v.to(dtype) for k, v in load_file(os.path.join(model_dir, "model.safetensors")).items()}
    return cfg, weights


# ---- parts ----------------------------------------------------------------------------------------------

def rms_norm(x: torch.Tensor, gain: torch.Tensor, eps: float) -> torch.Tensor:
    """main_models_new.py:38-42: (x * sqrt(D)) / (||x||_2 + eps) * scale; eps is added to the norm."""
    d = x.shape[-1]
    norm = torch.linalg.vector_norm(x, dim=-1, keepdim=True)
    return (x * math.sqrt(d)) / (norm + eps) * gain


def rope_tables(n_positions: int, head_dim: int, base: float, dtype=torch.float64):
    """main_models_new.py:63-69: theta_i = 1/base^(2i/hd); cos/sin of pos*theta, repeated twice along the last dim."""
    i = torch.arange(0, head_dim // 2, dtype=dtype)
    theta = 1.0 / torch.pow(torch.tensor(base, dtype=dtype), (2 * i) / head_dim)
    ang = torch.outer(torch.arange(n_positions, dtype=dtype), theta)
    return torch.cos(ang).repeat(1, 2), torch.sin(ang).repeat(1, 2)


def rotate_half(x: torch.Tensor) -> torch.Tensor:
    """main_models_new.py:71-73: cat(-x2, x1) of the two halves."""
    x1, x2 = x.chunk(2, dim=-1)
    return torch.cat((-x2, x1), dim=-1)


def apply_rope(x: torch.Tensor, positions: torch.Tensor, base: float) -> torch.Tensor:
    """main_models_new.py:75-80: x*cos + rotate_half(x)*sin at each row's position. x: (T, heads, hd)."""
    hd = x.shape[-1]
    cos, sin = rope_tables(int(positions.max()) + 1, hd, base, x.dtype)
    c, s = cos[positions].unsqueeze(1), sin[positions].unsqueeze(1)
    return x * c + rotate_half(x) * s


def causal_gqa_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, group: int,
                         window: int = 0) -> torch.Tensor:
    """q (T, NH, hd), k/v (T, KVH, hd) -> (T, NH, hd).

    Query head h uses key/value head h // group (paged_attention_kernels.py:49; the reference's own oracle
    repeats each kv head `group` times: test_server.py:40-42). Scores q.k / sqrt(hd)
    (paged_attention_kernels.py:214), row t sees keys j <= t (kv_len = pos + 1: server.py:231), softmax,
    weighted sum of values. window > 0 keeps only the keys j > t - window (not in the reference).
    """
    T, NH, hd = q.shape
    out = torch.empty_like(q)
    for h in range(NH):
        kh = k[:, h // group, :]
        vh = v[:, h // group, :]
        for t in range(T):
            lo = max(0, t - window + 1) if window > 0 else 0
            s = (kh[lo:t + 1] @ q[t, h]) / math.sqrt(hd)
            p = torch.softmax(s, dim=0)
            out[t, h] = p @ vh[lo:t + 1]
    return out


def swiglu_ffn(x, w1, w2, wfc):
    """main_models_new.py:51, 60: fc(silu(x@W1) * (x@W2)); weights stored [in, out]."""
    a = x @ w1
    return ((a * torch.sigmoid(a)) * (x @ w2)) @ wfc


def block(x, w: Dict[str, torch.Tensor], prefix: str, cfg, positions, window: int = 0):
    """main_models_new.py:117-136, 146-152: x + o(attn(rope(q,k), v)) with the norm inside; then x + ffn(norm(x))."""
    T, D = x.shape
    NH, G = cfg["n_heads"], cfg["group"]
    KVH, hd = NH // G, D // NH
    a = rms_norm(x, w[prefix + "att.rms_norm_att.scale"], cfg["eps"])
    q = (a @ w[prefix + "att.q_proj.weight"]).view(T, NH, hd)
    kv = (a @ w[prefix + "att.kv_proj.weight"]).view(T, 2, KVH, hd)     # main_models_new.py:126-127
    k, v = kv.unbind(1)
    q, k = apply_rope(q, positions, cfg["base"]), apply_rope(k, positions, cfg["base"])
    o = causal_gqa_attention(q, k, v, G, window).reshape(T, D)
    x = x + o @ w[prefix + "att.linear_proj.weight"]
    f = rms_norm(x, w[prefix + "rms_norm_ffn.scale"], cfg["eps"])
    return x + swiglu_ffn(f, w[prefix + "ffn.swig.linear1.weight"], w[prefix + "ffn.swig.linear2.weight"],
                          w[prefix + "ffn.fc.weight"])


def trunk_hidden(ids: Sequence[int], w, cfg) -> torch.Tensor:
    """main_models_new.py:212-217: embedding, every block, rms_out. Returns the normed hidden (T, D)."""
    t = torch.tensor(list(ids), dtype=torch.long)
    x = w["embedding.weight"][t]
    pos = torch.arange(len(ids))
    for l in range(cfg["n_layers"]):
        x = block(x, w, f"transformer_block_list.{l}.", cfg, pos)
    return rms_norm(x, w["rms_out.scale"], cfg["eps"])


def logits_of(h: torch.Tensor, w, cfg) -> torch.Tensor:
    """main_models_new.py:225-226: h @ E^T (tied); an untied table `lm_head.weight` (V, D) is this build's addition."""
    table = w["embedding.weight"] if cfg["tied"] else w["lm_head.weight"]
    return h @ table.T


def mtp_head_hidden(i: int, h_prev: torch.Tensor, ids: Sequence[int], w, cfg) -> torch.Tensor:
    """Head i over the whole sequence (server.py:336-359; main_models_new.py:163-171).

    Rows p in [0, T-1-i): input [h_prev[p] ; rms_embed(E[ids[p+1+i]])] @ proj, one block over the head's own
    rows at positions p, then the head's rms_out. h_prev is the previous stage's normed output.
    """
    T = len(ids)
    n = max(0, T - 1 - i)
    pre = f"mtp_heads_list.{i}."
    if n == 0:
        return h_prev[:0]
    tok = torch.tensor([ids[p + 1 + i] for p in range(n)], dtype=torch.long)
    e = rms_norm(w["embedding.weight"][tok], w[pre + "rms_embed.scale"], cfg["eps"])
    z = torch.cat([h_prev[:n], e], dim=-1) @ w[pre + "proj.weight"]
    z = block(z, w, pre + "trans_block.", cfg, torch.arange(n))
    return rms_norm(z, w[pre + "rms_out.scale"], cfg["eps"])


def forward_all(ids: Sequence[int], w, cfg):
    """(main logits (T, V), [head i logits (T-1-i, V)]). Head i's row p predicts token p+2+i."""
    h = trunk_hidden(ids, w, cfg)
    main = logits_of(h, w, cfg)
    heads = []
    prev = h
    for i in range(cfg["mtp"]):
        prev = mtp_head_hidden(i, prev, ids, w, cfg)
        heads.append(logits_of(prev, w, cfg))
    return main, heads


# ---- sampling -------------------------------------------------------------------------------------------

def sampling_probs(logits: torch.Tensor, temperature: float, top_k: int = 0, top_p: float = 0.0,
                   rep_penalty: float = 1.0, ctx: Optional[Sequence[int]] = None) -> torch.Tensor:
    """server.py:22-50 for one row: penalty -> temperature -> top-k -> top-p -> softmax."""
    l = logits.clone().double()
    if rep_penalty != 1.0 and ctx:
        for t in set(ctx):
            l[t] = l[t] / rep_penalty if l[t] > 0 else l[t] * rep_penalty
    l = l / temperature
    srt, idx = torch.sort(l, descending=True)
    V = l.numel()
    k = top_k if top_k > 0 else V
    srt[k:] = -math.inf
    pp = top_p if top_p > 0 else 2.0
    remove = torch.cumsum(torch.softmax(srt, dim=0), dim=0) > pp
    remove[1:] = remove[:-1].clone()
    remove[0] = False
    srt[remove] = -math.inf
    out = torch.full_like(l, -math.inf)
    out[idx] = srt
    return torch.softmax(out, dim=0)


def pick_by_uniform(probs: torch.Tensor, u: float) -> int:
    """Inverse of the cumulative distribution in token order: the first token whose running mass passes u."""
    c = torch.cumsum(probs.double(), dim=0)
    nz = torch.nonzero(c > u * float(c[-1]))
    return int(nz[0]) if len(nz) else int(torch.argmax(probs))


def greedy_generate(prompt: Sequence[int], n_new: int, w, cfg) -> List[int]:
    """No cache: recompute the whole sequence for every token, arg-max (top_k=1 in the reference: test_server.py:110)."""
    ids = list(prompt)
    for _ in range(n_new):
        h = trunk_hidden(ids, w, cfg)
        ids.append(int(torch.argmax(logits_of(h[-1:], w, cfg)[0])))
    return ids[len(prompt):]

"""Plain torch versions of the engine's operations, one function per kernel, with the kernels' signatures.

Two uses, both in tests only: as the reference that each HIP kernel is compared with, and as a stand-in
for the kernels so that the step function, the cache and the scheduler can be run on a machine without a
GPU. The engine never imports this file and has no CPU path of its own.
"""
from __future__ import annotations

import math

import torch


class TorchOps:
    def __init__(self, device="cpu", dtype=torch.float32, graphs=False):
        """graphs: let the engine keep steps in fixed buffers and "replay" them as it does with captured graphs on
        the GPU, only that a replay here is the same calls made again: the host side of that path without a device."""
        self.device = torch.device(device)
        self.dtype = dtype
        self.supports_graphs = self.emulates_graphs = bool(graphs)

    def empty(self, *shape, dtype=None):
        return torch.zeros(*shape, dtype=dtype or self.dtype, device=self.device)

    # ---- row-wise ---------------------------------------------------------------------------------------
    def embedding(self, table, tokens, out=None):
        r = table[tokens.long()]
        if out is not None:
            out[:tokens.numel()] = r
            return out
        return r

    def rmsnorm(self, x, gain, eps, out=None):
        xf = x.float()
        y = (xf * math.sqrt(x.shape[-1]) / (torch.linalg.vector_norm(xf, dim=-1, keepdim=True) + eps) * gain).to(x.dtype)
        if out is not None:
            out[:x.shape[0]] = y
            return out
        return y

    def embedding_rmsnorm(self, table, tokens, gain, eps, out=None):
        return self.rmsnorm(table[tokens.long()], gain, eps, out=out)

    def gather_rows(self, src, state, index, out=None):
        ix = index.long()
        rows = torch.zeros(ix.numel(), src.shape[1], dtype=src.dtype, device=src.device)
        from_src = ix >= 0
        rows[from_src] = src[ix[from_src]]
        rows[~from_src] = state[-ix[~from_src] - 1]
        if out is not None:
            out[:ix.numel()] = rows
            return out
        return rows

    def copy_rows(self, src, src_index, dst, dst_index):
        dst[dst_index.long()] = src[src_index.long()]

    def swiglu(self, gu, out=None):
        g, u = gu[:, 0::2].float(), gu[:, 1::2].float()      # gate and up columns come interleaved
        y = (g * torch.sigmoid(g) * u).to(gu.dtype)
        if out is not None:
            out.copy_(y)
            return out
        return y

    def linear(self, x, w, residual=None, out_dtype=None, rms=None, reuse_residual=False):
        if rms is not None:
            x = self.rmsnorm(x, rms[0], rms[1])
        y = x.float() @ w.float().t()
        if residual is not None:
            y = y + residual.float()
        return y.to(out_dtype or self.dtype)

    def linear_swiglu(self, x, w, rms=None):
        return self.swiglu(self.linear(x, w, rms=rms))

    # ---- rotary + cache write ---------------------------------------------------------------------------
    def qkv_rope(self, x, w, rms, positions, write_slots, table, plane, n_heads, n_kv_heads, head_dim, page_size,
                 interleaved=False, write_cache=True):
        qkv = self.linear(x, w, rms=rms)
        q = torch.zeros(x.shape[0], n_heads * head_dim, dtype=qkv.dtype, device=qkv.device)
        self.rope_write_kv(qkv, positions, write_slots, table, plane, n_heads, n_kv_heads, head_dim, page_size,
                           interleaved, write_cache, paired=True, q_out=q)
        return q

    def rope_write_kv(self, qkv, positions, write_slots, table, plane, n_heads, n_kv_heads, head_dim, page_size,
                      interleaved=False, write_cache=True, paired=False, q_out=None):
        n = qkv.shape[0]
        if n == 0:
            return
        qkv = qkv if not paired else qkv.clone()
        x = qkv.view(n, n_heads + 2 * n_kv_heads, head_dim)
        if paired:
            # pair j sits at columns 2j, 2j+1 of every q and k head: put the heads back in natural order first
            qk_p = x[:, :n_heads + n_kv_heads]
            first, second = qk_p[..., 0::2], qk_p[..., 1::2]
            nat = torch.stack((first, second), dim=-1).flatten(-2) if interleaved else torch.cat((first, second), dim=-1)
            x[:, :n_heads + n_kv_heads] = nat
        qk = x[:, :n_heads + n_kv_heads].float()
        if table is not None:
            cs = table[positions.long()]                     # [n, hd/2, 2]
            c, s = cs[..., 0].unsqueeze(1), cs[..., 1].unsqueeze(1)
            if interleaved:
                a, b = qk[..., 0::2], qk[..., 1::2]
                rot = torch.stack((a * c - b * s, b * c + a * s), dim=-1).flatten(-2)
            else:
                h = head_dim // 2
                a, b = qk[..., :h], qk[..., h:]
                rot = torch.cat((a * c - b * s, b * c + a * s), dim=-1)
            x[:, :n_heads + n_kv_heads] = rot.to(qkv.dtype)
        if q_out is not None:
            q_out.copy_(x[:, :n_heads].reshape(n, n_heads * head_dim))
        if write_cache:
            slots = write_slots.long()
            page, off = slots // page_size, slots % page_size
            # a page holds keys as [kv head][slot][head_dim] and values transposed, [kv head][head_dim][slot]
            plane[page, 0, :, off] = x[:, n_heads:n_heads + n_kv_heads]
            vt = plane[:, 1].reshape(plane.shape[0], n_kv_heads, head_dim, page_size)
            vt[page, :, :, off] = x[:, n_heads + n_kv_heads:]
            plane[:, 1] = vt.reshape(plane.shape[0], n_kv_heads, page_size, head_dim)

    # ---- attention over the paged cache -----------------------------------------------------------------
    def paged_attention(self, q, plane, batch, group, n_heads, n_kv_heads, head_dim, window=0, scale=None, slopes=None):
        n = q.shape[0]
        page_size = plane.shape[3]
        scale = scale if scale is not None else head_dim ** -0.5
        tables = batch.block_tables[group]
        g = n_heads // n_kv_heads
        out = torch.zeros(n, n_heads * head_dim, dtype=torch.float32, device=q.device)
        pos = batch.positions.tolist()
        seq = batch.row_seq.tolist()
        for r in range(n):
            p = pos[r]
            first = max(0, p - window + 1) if window > 0 else 0
            js = torch.arange(first, p + 1)
            pages = tables[seq[r]].long()[js // page_size]
            k = plane[pages, 0, :, js % page_size].float()       # [keys, kvh, hd]
            vt = plane[:, 1].reshape(plane.shape[0], n_kv_heads, head_dim, page_size)
            v = vt[pages, :, :, js % page_size].float()
            qr = q[r].float().view(n_heads, head_dim)
            for h in range(n_heads):
                s = (k[:, h // g] @ qr[h]) * scale
                if slopes is not None:
                    s = s + float(slopes[h]) * (js - p).float()
                out[r, h * head_dim:(h + 1) * head_dim] = torch.softmax(s, dim=0) @ v[:, h // g]
        return out.to(q.dtype)

    # ---- sampling ---------------------------------------------------------------------------------------
    def argmax(self, logits):
        return torch.argmax(logits, dim=-1).to(torch.int32)

    def sample(self, logits, temperature, top_k, top_p, rep_penalty, uniform, ctx_tokens=None, ctx_offsets=None,
               seen=None, seen_row=None):
        """The kernel's method: thresholds instead of a sort, inverse CDF in token order."""
        n, V = logits.shape
        out = torch.zeros(n, dtype=torch.int32)
        if seen is not None:
            # the byte-table form of the context: turn each row's line into a token list, mark the draw afterwards
            lists = [torch.nonzero(seen[int(seen_row[r])]).flatten().to(torch.int32) if int(seen_row[r]) >= 0
                     else torch.zeros(0, dtype=torch.int32) for r in range(n)]
            offs = torch.tensor([0] + list(torch.tensor([len(l) for l in lists]).cumsum(0)), dtype=torch.int32)
            flat = torch.cat(lists) if lists else torch.zeros(0, dtype=torch.int32)
            out = self.sample(logits, temperature, top_k, top_p, rep_penalty, uniform, flat, offs)
            for r in range(n):
                if int(seen_row[r]) >= 0:
                    seen[int(seen_row[r]), int(out[r])] = 1
            return out
        for r in range(n):
            l = logits[r].float().clone()
            t, k, p = float(temperature[r]), int(top_k[r]), float(top_p[r])
            pen = float(rep_penalty[r]) if rep_penalty is not None else 1.0
            greedy = t == 0.0 or k == 1
            inv_t = 1.0 if greedy else 1.0 / t
            x = l * inv_t
            if pen != 1.0 and ctx_tokens is not None:
                toks = ctx_tokens[int(ctx_offsets[r]):int(ctx_offsets[r + 1])].long().unique()
                lt = l[toks]
                x[toks] = torch.where(lt > 0, lt / pen, lt * pen) * inv_t
            if greedy:
                out[r] = int(torch.argmax(x))
                continue
            keep = torch.ones(V, dtype=torch.bool)
            if 0 < k < V:
                kth = torch.topk(x, k).values[-1]
                keep = x >= kth
            e = torch.where(keep, torch.exp(x - x.max()), torch.zeros_like(x))
            if 0.0 < p < 1.0:
                z = e.sum()
                order = torch.argsort(x, descending=True)
                before = torch.cumsum(e[order], 0) - e[order]
                ok = before <= p * z
                keep2 = torch.zeros(V, dtype=torch.bool)
                keep2[order[ok]] = True
                e = torch.where(keep2, e, torch.zeros_like(e))
            c = torch.cumsum(e.double(), 0)
            nz = torch.nonzero(c > float(uniform[r]) * float(c[-1]))
            out[r] = int(nz[0]) if len(nz) else int(torch.argmax(x))
        return out.to(logits.device)

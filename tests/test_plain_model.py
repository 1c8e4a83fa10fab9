"""What fixes the plain implementation beside the reference's text: special cases that reduce to a library routine,
invariants, and the vectors the reference's own tests hold. Each is chosen so that a plausible mistake fails it."""
import math

import pytest
import torch
import torch.nn.functional as F

import helpers as H
import plain_model as pm

torch.manual_seed(0)
D64 = torch.float64


# ---- RMSNorm (main_models_new.py:31-42) ---------------------------------------------------------------------

def test_rmsnorm_reduces_to_the_library_norm_without_eps():
    x, g = torch.randn(5, 48, dtype=D64), 1 + 0.1 * torch.randn(48, dtype=D64)
    torch.testing.assert_close(pm.rms_norm(x, g, 0.0), F.rms_norm(x, (48,), g, eps=0.0))


def test_rmsnorm_invariants_and_eps_outside_the_root():
    x = torch.randn(4, 32, dtype=D64)
    ones = torch.ones(32, dtype=D64)
    y = pm.rms_norm(x, ones, 2e-8)
    torch.testing.assert_close(y.norm(dim=-1), torch.full((4,), math.sqrt(32), dtype=D64))
    torch.testing.assert_close(pm.rms_norm(7.5 * x, ones, 0.0), pm.rms_norm(x, ones, 0.0))
    assert torch.equal(pm.rms_norm(torch.zeros(1, 32, dtype=D64), ones, 2e-8), torch.zeros(1, 32, dtype=D64))
    # eps is added to the norm itself: a row whose norm equals eps comes out at half the full size;
    # rsqrt(mean(x^2) + eps) would leave it at 1e-4 of it or at full size
    tiny = torch.zeros(1, 32, dtype=D64); tiny[0, 0] = 1e-3
    assert pm.rms_norm(tiny, ones, 1e-3).norm().item() == pytest.approx(math.sqrt(32) / 2)


# ---- rotary (main_models_new.py:63-80) -----------------------------------------------------------------------

def test_rope_identity_norm_and_pairing():
    x = torch.randn(3, 2, 16, dtype=D64)
    torch.testing.assert_close(pm.apply_rope(x, torch.zeros(3, dtype=torch.long), 1e4), x)
    y = pm.apply_rope(x, torch.tensor([5, 17, 100]), 1e4)
    torch.testing.assert_close(y.norm(dim=-1), x.norm(dim=-1))
    e0 = torch.zeros(1, 1, 16, dtype=D64); e0[0, 0, 0] = 1
    r = pm.apply_rope(e0, torch.tensor([1]), 1e4)[0, 0]
    # the pair of index 0 is index head_dim/2 (half split, not interleaved), theta_0 = 1, and the sine is positive
    assert r[0].item() == pytest.approx(math.cos(1)) and r[8].item() == pytest.approx(math.sin(1))
    assert r[1].abs().item() < 1e-12
    e1 = torch.zeros(1, 1, 16, dtype=D64); e1[0, 0, 1] = 1
    th = 1e4 ** (-2 / 16)
    r = pm.apply_rope(e1, torch.tensor([3]), 1e4)[0, 0]
    assert r[1].item() == pytest.approx(math.cos(3 * th)) and r[9].item() == pytest.approx(math.sin(3 * th))


def test_rope_scores_depend_on_distance_only():
    q, k = torch.randn(1, 1, 32, dtype=D64), torch.randn(1, 1, 32, dtype=D64)
    def score(m, n):
        return (pm.apply_rope(q, torch.tensor([m]), 5e5) * pm.apply_rope(k, torch.tensor([n]), 5e5)).sum().item()
    assert score(9, 4) == pytest.approx(score(109, 104)) and score(9, 4) == pytest.approx(score(5, 0))
    assert abs(score(9, 4) - score(4, 9)) > 1e-6


# ---- attention (paged_attention_kernels.py:49, 86-108; test_server.py:33-43) ---------------------------------

def test_attention_special_cases_reduce_to_library_attention():
    T, NH, hd = 9, 4, 8
    q, k, v = (torch.randn(T, NH, hd, dtype=D64) for _ in range(3))
    lib = F.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1), is_causal=True)
    torch.testing.assert_close(pm.causal_gqa_attention(q, k, v, 1), lib.transpose(0, 1))
    # one key: the output is that key's value
    torch.testing.assert_close(pm.causal_gqa_attention(q[:1], k[:1], v[:1], 1), v[:1])
    # one head
    lib1 = F.scaled_dot_product_attention(q[:, :1].transpose(0, 1), k[:, :1].transpose(0, 1), v[:, :1].transpose(0, 1), is_causal=True)
    torch.testing.assert_close(pm.causal_gqa_attention(q[:, :1], k[:, :1], v[:, :1], 1), lib1.transpose(0, 1))


def test_gqa_head_mapping_is_h_div_group():
    """The reference's oracle repeats each kv head `group` times (test_server.py:40-42; test_gqa_paged.py:39-44);
    passing the number of kv heads as the group size must not match (test_gqa_paged.py:50-53)."""
    T, NH, KVH, hd = 7, 8, 2, 16
    G = NH // KVH
    q, k, v = torch.randn(T, NH, hd, dtype=D64), torch.randn(T, KVH, hd, dtype=D64), torch.randn(T, KVH, hd, dtype=D64)
    kq, vq = k.repeat_interleave(G, dim=1), v.repeat_interleave(G, dim=1)
    lib = F.scaled_dot_product_attention(q.transpose(0, 1), kq.transpose(0, 1), vq.transpose(0, 1), is_causal=True).transpose(0, 1)
    got = pm.causal_gqa_attention(q, k, v, G)
    torch.testing.assert_close(got, lib)
    wrong = F.scaled_dot_product_attention(q.transpose(0, 1), k.repeat(1, G, 1).transpose(0, 1),
                                           v.repeat(1, G, 1).transpose(0, 1), is_causal=True).transpose(0, 1)   # h % KVH
    assert not torch.allclose(got, wrong, atol=1e-3)


def test_attention_window():
    T, hd = 12, 8
    q, k, v = (torch.randn(T, 1, hd, dtype=D64) for _ in range(3))
    full = pm.causal_gqa_attention(q, k, v, 1)
    torch.testing.assert_close(pm.causal_gqa_attention(q, k, v, 1, window=T), full)
    w = pm.causal_gqa_attention(q, k, v, 1, window=3)
    torch.testing.assert_close(w[:3], full[:3])
    torch.testing.assert_close(w[7:8], pm.causal_gqa_attention(q[5:8], k[5:8], v[5:8], 1)[2:3])


# ---- feed-forward, block, trunk --------------------------------------------------------------------------------

def test_swiglu():
    x, w1, w2, wf = torch.randn(3, 8, dtype=D64), torch.randn(8, 20, dtype=D64), torch.randn(8, 20, dtype=D64), torch.randn(20, 8, dtype=D64)
    torch.testing.assert_close(pm.swiglu_ffn(x, w1, w2, wf), (F.silu(x @ w1) * (x @ w2)) @ wf)
    w1z = w1.clone(); w1z[:, 4] = 0                 # a zero gate column removes that hidden unit, whatever the up half holds
    wfz = wf.clone(); wfz[4] = 0
    torch.testing.assert_close(pm.swiglu_ffn(x, w1z, w2, wf), pm.swiglu_ffn(x, w1, w2, wfz))


@pytest.fixture(scope="module")
def model_b():
    return pm.read_model_folder(H.model_folder("B", "float32"))


def test_block_residuals_pass_the_stream_unnormed(model_b):
    cfg, w = model_b
    w = dict(w)
    pre = "transformer_block_list.0."
    w[pre + "att.linear_proj.weight"] = torch.zeros_like(w[pre + "att.linear_proj.weight"])
    w[pre + "ffn.fc.weight"] = torch.zeros_like(w[pre + "ffn.fc.weight"])
    x = torch.randn(5, cfg["d_model"], dtype=D64) * 3
    torch.testing.assert_close(pm.block(x, w, pre, cfg, torch.arange(5)), x)


def test_positions_shifted_together_change_nothing(model_b):
    cfg, w = model_b
    x = torch.randn(6, cfg["d_model"], dtype=D64)
    a = pm.block(x, w, "transformer_block_list.1.", cfg, torch.arange(6))
    b = pm.block(x, w, "transformer_block_list.1.", cfg, torch.arange(6) + 37)
    torch.testing.assert_close(a, b)


def test_causality_and_gains(model_b):
    cfg, w = model_b
    ids = H.random_ids(cfg["vocab"], 12, 1)
    h = pm.trunk_hidden(ids, w, cfg)
    ids2 = list(ids); ids2[8] = (ids2[8] + 1) % cfg["vocab"]
    h2 = pm.trunk_hidden(ids2, w, cfg)
    torch.testing.assert_close(h[:8], h2[:8])
    assert not torch.allclose(h[8:], h2[8:], atol=1e-4)
    # a dropped gain shows: the folder's gains are not 1
    w2 = dict(w); w2["rms_out.scale"] = torch.ones_like(w["rms_out.scale"])
    assert not torch.allclose(pm.trunk_hidden(ids, w2, cfg), h, atol=1e-3)


# ---- prediction heads (server.py:336-359; main_models_new.py:163-171) ------------------------------------------

def test_head_rows_and_what_they_depend_on(model_b):
    cfg, w = model_b
    ids = H.random_ids(cfg["vocab"], 11, 2)
    main, heads = pm.forward_all(ids, w, cfg)
    assert main.shape[0] == 11 and [h.shape[0] for h in heads] == [10, 9]        # head i has T-1-i rows
    for i in (0, 1):
        p = 4
        later = list(ids); later[p + 2 + i] = (later[p + 2 + i] + 1) % cfg["vocab"]
        torch.testing.assert_close(pm.forward_all(later, w, cfg)[1][i][:p + 1], heads[i][:p + 1])
        at = list(ids); at[p + 1 + i] = (at[p + 1 + i] + 1) % cfg["vocab"]        # the token whose embedding it eats
        assert not torch.allclose(pm.forward_all(at, w, cfg)[1][i][p], heads[i][p], atol=1e-4)
    assert pm.forward_all(ids[:1], w, cfg)[1][0].shape[0] == 0                   # a one-token prompt: no head rows


def test_head_fusion_order_and_norms(model_b):
    """The first d_model rows of proj meet the previous stage's output, which gets no norm of its own; only the
    embedding is normed (main_models_new.py:164)."""
    cfg, w = model_b
    D = cfg["d_model"]
    ids = H.random_ids(cfg["vocab"], 6, 3)
    h = pm.trunk_hidden(ids, w, cfg)
    base = pm.mtp_head_hidden(0, h, ids, w, cfg)
    w2 = dict(w); p = w["mtp_heads_list.0.proj.weight"].clone(); p[D:] = 0; w2["mtp_heads_list.0.proj.weight"] = p
    ids_other = [ids[0]] + [(t + 5) % cfg["vocab"] for t in ids[1:]]
    torch.testing.assert_close(pm.mtp_head_hidden(0, h, ids, w2, cfg), pm.mtp_head_hidden(0, h, ids_other, w2, cfg))
    assert not torch.allclose(pm.mtp_head_hidden(0, 2 * h, ids, w2, cfg), pm.mtp_head_hidden(0, h, ids, w2, cfg), atol=1e-4)
    w3 = dict(w); p = w["mtp_heads_list.0.proj.weight"].clone(); p[:D] = 0; w3["mtp_heads_list.0.proj.weight"] = p
    w3["embedding.weight"] = 3 * w["embedding.weight"]           # scaling the embedding is undone by its norm
    w3n = dict(w3); w3n["embedding.weight"] = w["embedding.weight"]
    # (up to eps / ||e||: this folder's eps is 1e-5 and an embedding's norm about 0.5)
    torch.testing.assert_close(pm.mtp_head_hidden(0, h, ids, w3, cfg), pm.mtp_head_hidden(0, h, ids, w3n, cfg),
                               atol=2e-4, rtol=0)
    assert base.shape == (5, D)


# ---- sampling (server.py:22-50) --------------------------------------------------------------------------------

def test_repetition_penalty_vector_of_the_reference():
    """test_server.py:120-122."""
    lg = torch.zeros(100); lg[5] = 5.0; lg[7] = 4.9
    assert pm.sampling_probs(lg, 1.0).argmax().item() == 5
    assert pm.sampling_probs(lg, 1.0, rep_penalty=2.0, ctx=[5]).argmax().item() == 7
    neg = torch.zeros(10); neg[3] = -1.0
    assert pm.sampling_probs(neg, 1.0, rep_penalty=2.0, ctx=[3, 3])[3].item() == pytest.approx(
        math.exp(-2.0) / (9 + math.exp(-2.0)))


def test_top_k_and_top_p():
    lg = torch.log(torch.tensor([0.5, 0.3, 0.15, 0.05]))
    assert pm.sampling_probs(lg, 1.0, top_k=1).tolist() == [1.0, 0.0, 0.0, 0.0]
    torch.testing.assert_close(pm.sampling_probs(lg, 1.0, top_k=2), torch.tensor([0.625, 0.375, 0, 0], dtype=D64))
    # top_p keeps the token that crosses p: 0.5 < 0.6 so the second stays, the third goes
    torch.testing.assert_close(pm.sampling_probs(lg, 1.0, top_p=0.6), torch.tensor([0.625, 0.375, 0, 0], dtype=D64))
    torch.testing.assert_close(pm.sampling_probs(lg, 1.0, top_p=0.8), torch.tensor([0.625, 0.375, 0, 0], dtype=D64))
    torch.testing.assert_close(pm.sampling_probs(lg, 1.0, top_p=0.81)[:3], torch.tensor([0.5, 0.3, 0.15], dtype=D64) / 0.95)
    torch.testing.assert_close(pm.sampling_probs(lg, 0.5)[0], torch.tensor(0.25 / (0.25 + 0.09 + 0.0225 + 0.0025), dtype=D64))


def test_inverse_cdf_draw_follows_the_probabilities():
    probs = torch.tensor([0.1, 0.0, 0.6, 0.3], dtype=D64)
    assert [pm.pick_by_uniform(probs, u) for u in (0.0, 0.0999, 0.1, 0.69, 0.7, 0.999)] == [0, 0, 2, 2, 3, 3]
    n = 4000
    counts = torch.zeros(4)
    for i in range(n):
        counts[pm.pick_by_uniform(probs, (i + 0.5) / n)] += 1
    torch.testing.assert_close(counts / n, probs.float(), atol=1e-3, rtol=0)

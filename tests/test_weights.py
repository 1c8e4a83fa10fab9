"""Weights by name from safetensors: what is kept, and the one error that lists everything that is wrong."""
import os

import pytest
import torch
from safetensors.torch import load_file, save_file

import helpers as H
from tiny_inference_server_amd.config import ARCHITECTURES, load_config
from tiny_inference_server_amd.weights import WeightError, load_tensors, random_tensors, spec_tensors, write_random_model


def spec_of(folder):
    cfg = load_config(folder)
    return ARCHITECTURES.get(cfg.architecture).build_spec(cfg)


def test_random_model_folder_loads_and_is_seeded(tmp_path):
    cfg = H.TINY["B"]["cfg"]
    d1 = write_random_model(cfg, 5, str(tmp_path / "one"), gain_jitter=0.1)
    d2 = write_random_model(cfg, 5, str(tmp_path / "two"), gain_jitter=0.1)
    d3 = write_random_model(cfg, 6, str(tmp_path / "three"), gain_jitter=0.1)
    assert sorted(os.listdir(d1)) == ["config.json", "model.safetensors"]
    t1, t2, t3 = (load_tensors(d, spec_of(d)) for d in (d1, d2, d3))
    assert set(t1) == set(spec_tensors(spec_of(d1)))
    assert all(torch.equal(t1[k], t2[k]) for k in t1) and any(not torch.equal(t1[k], t3[k]) for k in t1)
    assert all(v.dtype == torch.bfloat16 for v in t1.values())
    w = t1["transformer_block_list.0.att.q_proj.weight"].float()
    assert abs(w.std().item() - 0.02) < 2e-3 and abs(w.mean().item()) < 2e-3
    assert "lm_head.weight" in t1 and t1["lm_head.weight"].shape == (cfg.vocab_size, cfg.d_model)
    # reference shapes: q (D, D), kv (D, 2D/G), fc (F, D), proj (2D, D)   (main_models_new.py:86-89, 56-57, 158)
    D, G, F = cfg.d_model, cfg.group_size, cfg.ffn_hidden
    assert t1["transformer_block_list.2.att.kv_proj.weight"].shape == (D, 2 * D // G)
    assert t1["transformer_block_list.2.ffn.fc.weight"].shape == (F, D)
    assert t1["mtp_heads_list.1.proj.weight"].shape == (2 * D, D)


def test_stored_precision_is_kept(tmp_path):
    cfg = H.TINY["A"]["cfg"]
    d = write_random_model(cfg, 1, str(tmp_path / "m"))
    path = os.path.join(d, "model.safetensors")
    t = load_file(path)
    t["rms_out.scale"] = t["rms_out.scale"].float() * 1.00001          # a tensor stored in 32 bits stays 32-bit
    t["embedding.weight"] = t["embedding.weight"].to(torch.float16)     # 16-bit floats are kept as bfloat16
    t["cos"] = torch.zeros(4, 8)                                        # the reference's derived buffers may be present
    t["transformer_block_list.0.att.rms_norm_att.eps"] = torch.tensor(2e-8)
    save_file(t, path)
    got = load_tensors(d, spec_of(d))
    assert got["rms_out.scale"].dtype == torch.float32 and got["rms_out.scale"][0].item() == pytest.approx(1.00001)
    assert got["embedding.weight"].dtype == torch.bfloat16
    assert "cos" not in got


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    cfg = H.TINY["A"]["cfg"]
    d = write_random_model(cfg, 1, str(tmp_path / "m"))
    path = os.path.join(d, "model.safetensors")
    t = load_file(path)
    del t["rms_out.scale"], t["transformer_block_list.1.ffn.fc.weight"]
    t["lm_head.weight"] = torch.zeros(cfg.vocab_size, cfg.d_model)               # tied model with a stray output table
    t["transformer_block_list.0.att.kv_proj.weight"] = torch.zeros(cfg.d_model, cfg.d_model)     # as if G were 2
    t["extra.bias"] = torch.zeros(3)
    save_file(t, path)
    with pytest.raises(WeightError) as e:
        load_tensors(d, spec_of(d))
    msg = str(e.value)
    assert "missing tensors (2): rms_out.scale, transformer_block_list.1.ffn.fc.weight" in msg
    assert "unexpected tensors (2): extra.bias, lm_head.weight" in msg
    assert "wrong shapes (1): transformer_block_list.0.att.kv_proj.weight is [64, 64], expected [64, 32]" in msg


def test_missing_file(tmp_path):
    cfg = H.TINY["A"]["cfg"]
    d = write_random_model(cfg, 1, str(tmp_path / "m"))
    os.remove(os.path.join(d, "model.safetensors"))
    with pytest.raises(WeightError, match="no model.safetensors"):
        load_tensors(d, spec_of(d))


def test_random_tensors_gains_and_storage():
    cfg = H.TINY["A"]["cfg"]
    plain = random_tensors(cfg, 3, dtype="float32")
    assert all(torch.equal(v, torch.ones_like(v)) for k, v in plain.items() if v.dim() == 1)
    jit = random_tensors(cfg, 3, gain_jitter=0.1, dtype="float32")
    assert any(not torch.equal(v, torch.ones_like(v)) for k, v in jit.items() if v.dim() == 1)
    assert all(v.dtype == torch.float32 for v in plain.values())


def test_parameter_count_of_the_reference_model():
    """README.md:99-102 of the reference: 817M in the main model, 59M in the two heads, with the 48,011-token table."""
    from tiny_inference_server_amd.config import config_from_dict
    cfg = config_from_dict({"architecture": "GqaMtpTransformer", "D_MODEL": 1536, "VOCAB_SIZE": 48011,
                            "MAX_CONTEXT": 8192, "MAX_FREQ": 10000, "N_HEAD": 12, "NUM_LAYERS": 30,
                            "FFN_HIDDEN_DIM": 4096, "NUM_GROUPS": 4, "MTP_HEADS": 2})
    shapes = spec_tensors(ARCHITECTURES.get(cfg.architecture).build_spec(cfg))
    count = lambda pred: sum(int(torch.tensor(s).prod()) for n, s in shapes.items() if pred(n))
    heads = count(lambda n: n.startswith("mtp_heads_list."))
    trunk = count(lambda n: not n.startswith("mtp_heads_list."))
    assert round(trunk / 1e6) == 817 and round(heads / 1e6) == 59

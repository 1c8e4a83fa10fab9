"""Configuration: the reference's field names as config.json keys, the registry, and the errors."""
import json
import os

import pytest

from tiny_inference_server_amd import architectures  # noqa: F401
from tiny_inference_server_amd.config import (ARCHITECTURES, ConfigError, GqaMtpConfig, Registry, config_from_dict,
                                              load_config, save_config)

REF = {"architecture": "GqaMtpTransformer", "D_MODEL": 1536, "VOCAB_SIZE": 48011, "MAX_CONTEXT": 8192,
       "MAX_FREQ": 10000, "N_HEAD": 12, "NUM_LAYERS": 30, "FFN_HIDDEN_DIM": 4096, "NUM_GROUPS": 4, "MTP_HEADS": 2}


def test_reference_field_names_are_the_keys():
    """The values of reference Config/config.py:11-23 give the 0.9B model; NUM_GROUPS is the group size."""
    c = config_from_dict(REF)
    assert (c.d_model, c.vocab_size, c.max_context, c.n_heads, c.n_layers, c.ffn_hidden) == (1536, 48011, 8192, 12, 30, 4096)
    assert c.group_size == 4 and c.n_kv_heads == 3 and c.head_dim == 128 and c.mtp_heads == 2
    assert c.rope_base == 10000.0 and c.rms_eps == 2e-8 and c.tie_embeddings and c.eos_token_id == -1


def test_aliases_defaults_and_extra_keys():
    raw = {"architecture": "GqaMtpTransformer", "d_model": 96, "vocab_size": 1000, "max_context": 64,
           "rope_base": 5e5, "n_heads": 3, "n_layers": 3, "ffn_hidden": 256, "n_kv_heads": 1,
           "RMS_EPS": 1e-5, "TIE_EMBEDDINGS": False, "EOS": 7, "BATCH_SIZE": 24}
    c = config_from_dict(raw)
    assert c.group_size == 3 and c.mtp_heads == 0 and c.rms_eps == 1e-5 and not c.tie_embeddings and c.eos_token_id == 7
    assert c.extra == {"BATCH_SIZE": 24}


def test_round_trip_through_a_folder(tmp_path):
    c = config_from_dict(REF)
    save_config(c, str(tmp_path))
    assert json.load(open(os.path.join(tmp_path, "config.json")))["NUM_GROUPS"] == 4
    assert load_config(str(tmp_path)) == c


@pytest.mark.parametrize("change,needle", [
    ({"D_MODEL": None}, "lacks 'D_MODEL'"),
    ({"NUM_GROUPS": None}, "lacks 'NUM_GROUPS'"),
    ({"architecture": None}, "lacks 'architecture'"),
    ({"architecture": "Llama"}, "unknown architecture 'Llama'; known: GqaMtpTransformer"),
    ({"N_HEAD": 7}, "not a multiple of n_heads"),
    ({"NUM_GROUPS": 5}, "not a multiple of the group size"),
    ({"D_MODEL": 36, "N_HEAD": 12}, "must be even"),
    ({"NUM_LAYERS": 0}, "n_layers must be at least 1"),
    ({"D_MODEL": "big"}, "must be an integer"),
    ({"TIE_EMBEDDINGS": 1}, "must be true or false"),
    ({"MAX_FREQ": -1}, "rotary base must be positive"),
    ({"MAX_CONTEXT": 3}, "leaves no room"),
])
def test_errors_name_the_key(change, needle):
    raw = dict(REF)
    for k, v in change.items():
        if v is None:
            raw.pop(k)
        else:
            raw[k] = v
    with pytest.raises(ConfigError) as e:
        config_from_dict(raw)
    assert needle in str(e.value)


def test_missing_folder_and_bad_json(tmp_path):
    with pytest.raises(ConfigError, match="no config.json"):
        load_config(str(tmp_path))
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(ConfigError, match="not valid JSON"):
        load_config(str(tmp_path))


def test_registry():
    r = Registry("thing")
    r.register("a", 1)

    @r.register("b")
    def b():
        return 2
    assert r.get("a") == 1 and r.get("b") is b and "a" in r and list(r) == ["a", "b"]
    with pytest.raises(KeyError, match="already registered"):
        r.register("a", 3)
    r.register("a", 3, replace=True)
    with pytest.raises(KeyError, match="unknown thing 'c'; known: a, b"):
        r.get("c")
    assert "GqaMtpTransformer" in ARCHITECTURES


def test_spec_is_built_from_the_config_alone():
    """Every size in the spec comes from the configuration: two configurations, two different specs."""
    a = GqaMtpConfig(d_model=64, vocab_size=512, max_context=256, rope_base=1e4, n_heads=8, n_layers=2, ffn_hidden=176,
                     group_size=4, mtp_heads=1)
    b = GqaMtpConfig(d_model=96, vocab_size=1000, max_context=128, rope_base=5e5, n_heads=3, n_layers=3,
                     ffn_hidden=256, group_size=3, mtp_heads=2, rms_eps=1e-5, tie_embeddings=False)
    build = ARCHITECTURES.get("GqaMtpTransformer").build_spec
    sa, sb = build(a), build(b)
    assert len(sa.layers) == 3 and len(sb.layers) == 5 and [s.lag for s in sb.stages] == [0, 1, 2]
    assert sa.lm_head == sa.embedding and sb.lm_head == "lm_head.weight"
    ma, mb = sa.layers[0].part("mixer").params, sb.layers[0].part("mixer").params
    assert (ma["n_heads"], ma["n_kv_heads"], ma["head_dim"]) == (8, 2, 8)
    assert (mb["n_heads"], mb["n_kv_heads"], mb["head_dim"]) == (3, 1, 32)
    assert ma["position"].params["base"] == 1e4 and mb["position"].params["base"] == 5e5
    assert sa.layers[0].part("mixer_norm").params["eps"] == 2e-8 and sb.layers[0].part("mixer_norm").params["eps"] == 1e-5
    assert sb.layers[4].part("mixer").tensors["q"] == "mtp_heads_list.1.trans_block.att.q_proj.weight"

"""The grouped-query decoder with multi-token-prediction heads, as a spec of parts.

Trunk: token embedding -> n_layers pre-norm blocks (RMSNorm, rotary grouped-query attention, SwiGLU) ->
RMSNorm -> output table, tied to the embedding or not (reference main_models_new.py:174-226).
Prediction head i: [previous stage's normed output ; RMSNorm(E[token p+1+i])] . proj -> one more block with
a cache of its own -> RMSNorm -> the same output table (main_models_new.py:155-171; server.py:336-359).
Head i at position p consumes the token p+1+i, so as a stage it lags the tokens by i+1 positions.

Tensor names are the reference's state-dict names; `lm_head.weight` (vocab, d_model) exists when the
output table is not tied. A file may also carry the reference's derived buffers, which are not read.
"""
from __future__ import annotations

from ..config.model_config import ARCHITECTURES, Architecture, GqaMtpConfig
from ..parts.spec import LayerCall, LayerSpec, ModelSpec, PartSpec, StageSpec


def _norm(cfg, name):
    return PartSpec("norm", "rmsnorm_l2", {"width": cfg.d_model, "eps": cfg.rms_eps}, {"gain": name})


def _block(cfg, prefix):
    position = PartSpec("position", "rotary", {"head_dim": cfg.head_dim, "base": cfg.rope_base,
                                               "max_context": cfg.max_context, "pairing": "half"})
    mixer = PartSpec("mixer", "gqa_attention",
                     {"d_model": cfg.d_model, "n_heads": cfg.n_heads, "n_kv_heads": cfg.n_kv_heads,
                      "head_dim": cfg.head_dim, "window": 0, "position": position},
                     {"q": prefix + "att.q_proj.weight", "kv": prefix + "att.kv_proj.weight",
                      "o": prefix + "att.linear_proj.weight"})
    ffn = PartSpec("feed_forward", "swiglu", {"d_model": cfg.d_model, "hidden": cfg.ffn_hidden},
                   {"gate": prefix + "ffn.swig.linear1.weight", "up": prefix + "ffn.swig.linear2.weight",
                    "down": prefix + "ffn.fc.weight"})
    return LayerSpec("prenorm_residual", {"mixer_norm": _norm(cfg, prefix + "att.rms_norm_att.scale"), "mixer": mixer,
                                          "feed_forward_norm": _norm(cfg, prefix + "rms_norm_ffn.scale"),
                                          "feed_forward": ffn})


def build_spec(cfg: GqaMtpConfig) -> ModelSpec:
    layers = [_block(cfg, f"transformer_block_list.{l}.") for l in range(cfg.n_layers)]
    stages = [StageSpec(name="trunk", lag=0, input=PartSpec("stage_input", "token_embedding"),
                        calls=tuple(LayerCall(l) for l in range(cfg.n_layers)),
                        out_norm=_norm(cfg, "rms_out.scale"))]
    for i in range(cfg.mtp_heads):
        prefix = f"mtp_heads_list.{i}."
        layers.append(_block(cfg, prefix + "trans_block."))
        fuse = PartSpec("stage_input", "fuse_previous_stage",
                        {"d_model": cfg.d_model, "embed_norm": _norm(cfg, prefix + "rms_embed.scale")},
                        {"proj": prefix + "proj.weight"})
        stages.append(StageSpec(name=f"mtp{i}", lag=i + 1, input=fuse,
                                calls=(LayerCall(cfg.n_layers + i),),
                                out_norm=_norm(cfg, prefix + "rms_out.scale"),
                                state_key=f"mtp{i}.input"))
    return ModelSpec(
        d_model=cfg.d_model, vocab_size=cfg.vocab_size, max_context=cfg.max_context,
        layers=tuple(layers), stages=tuple(stages),
        embedding="embedding.weight",
        lm_head="embedding.weight" if cfg.tie_embeddings else "lm_head.weight",
        eos_token_id=cfg.eos_token_id,
        ignorable=("cos", "sin", "*.rootn", "*.eps"),
    )


ARCHITECTURES.register("GqaMtpTransformer", Architecture("GqaMtpTransformer", GqaMtpConfig, build_spec))

"""Typed model configuration read from a model folder's config.json.

The reference keeps its sizes in an UPPER_CASE dataclass shared with training
(reference Config/config.py:5-23) and has no config.json; a model folder here
carries those same field names as JSON keys.  The model fields are D_MODEL,
VOCAB_SIZE, MAX_CONTEXT, MAX_FREQ (the rotary base), N_HEAD, NUM_LAYERS,
FFN_HIDDEN_DIM, NUM_GROUPS (the number of query heads per key/value head:
reference main_models_new.py:92) and MTP_HEADS.  Three more keys name what the
reference fixes in code: RMS_EPS (main_models_new.py:36), TIE_EMBEDDINGS
(main_models_new.py:225-226) and EOS (server.py:12).

`architecture` selects the entry of the architecture registry; each entry
brings its own configuration class, so another architecture reads its own keys.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field, fields
from typing import Any, Callable, Dict, Mapping

from .registry import Registry


class ConfigError(ValueError):
    pass


@dataclass(frozen=True)
class Architecture:
    """What the registry holds for one architecture name."""
    name: str
    config_class: type                      # has from_dict(mapping) and to_dict()
    build_spec: Callable[[Any], Any]        # config -> ModelSpec (parts, layers, stages)


ARCHITECTURES: Registry[Architecture] = Registry("architecture")


def _take(raw: Mapping[str, Any], names, kind, default=None, required=True):
    """First of `names` present in `raw`, converted to `kind`."""
    for n in names:
        if n in raw:
            v = raw[n]
            if kind is bool:
                if not isinstance(v, bool):
                    raise ConfigError(f"config key {n!r} must be true or false, got {v!r}")
                return v
            if kind is int:
                if isinstance(v, bool) or not isinstance(v, int):
                    if isinstance(v, float) and v == int(v):
                        return int(v)
                    raise ConfigError(f"config key {n!r} must be an integer, got {v!r}")
                return v
            if kind is float:
                if isinstance(v, bool) or not isinstance(v, (int, float)):
                    raise ConfigError(f"config key {n!r} must be a number, got {v!r}")
                return float(v)
            return kind(v)
    if required:
        raise ConfigError(f"config.json lacks {names[0]!r}" +
                          (f" (also read as {', '.join(map(repr, names[1:]))})" if len(names) > 1 else ""))
    return default


@dataclass(frozen=True)
class GqaMtpConfig:
    """Sizes and constants of the grouped-query decoder with multi-token-prediction heads."""
    d_model: int
    vocab_size: int
    max_context: int
    rope_base: float
    n_heads: int
    n_layers: int
    ffn_hidden: int
    group_size: int            # query heads per key/value head (the reference's NUM_GROUPS)
    mtp_heads: int = 0
    rms_eps: float = 2e-8      # reference main_models_new.py:36
    tie_embeddings: bool = True
    eos_token_id: int = -1     # -1: no end-of-sequence token
    architecture: str = "GqaMtpTransformer"
    extra: Dict[str, Any] = field(default_factory=dict, compare=False)

    # key in config.json (reference name first), then accepted aliases
    KEYS = {
        "d_model": ("D_MODEL", "d_model"),
        "vocab_size": ("VOCAB_SIZE", "vocab_size"),
        "max_context": ("MAX_CONTEXT", "max_context"),
        "rope_base": ("MAX_FREQ", "rope_base"),
        "n_heads": ("N_HEAD", "n_heads"),
        "n_layers": ("NUM_LAYERS", "n_layers"),
        "ffn_hidden": ("FFN_HIDDEN_DIM", "ffn_hidden"),
        "group_size": ("NUM_GROUPS", "group_size"),
        "mtp_heads": ("MTP_HEADS", "mtp_heads"),
        "rms_eps": ("RMS_EPS", "rms_eps"),
        "tie_embeddings": ("TIE_EMBEDDINGS", "tie_embeddings"),
        "eos_token_id": ("EOS", "eos_token_id"),
    }

    @property
    def n_kv_heads(self) -> int:
        return self.n_heads // self.group_size

    @property
    def head_dim(self) -> int:
        return self.d_model // self.n_heads

    def __post_init__(self):
        def need(cond, msg):
            if not cond:
                raise ConfigError(msg)
        for name in ("d_model", "vocab_size", "max_context", "n_heads", "n_layers", "ffn_hidden", "group_size"):
            need(getattr(self, name) >= 1, f"{name} must be at least 1, got {getattr(self, name)}")
        need(self.mtp_heads >= 0, f"mtp_heads must not be negative, got {self.mtp_heads}")
        need(self.d_model % self.n_heads == 0,
             f"d_model {self.d_model} is not a multiple of n_heads {self.n_heads}")
        need(self.n_heads % self.group_size == 0,
             f"n_heads {self.n_heads} is not a multiple of the group size {self.group_size} (NUM_GROUPS)")
        need(self.head_dim % 2 == 0, f"head size {self.head_dim} must be even for the rotary pairs")
        need(self.rope_base > 0, f"rotary base must be positive, got {self.rope_base}")
        need(self.rms_eps >= 0, f"rms_eps must not be negative, got {self.rms_eps}")
        need(self.max_context > self.mtp_heads + 2,
             f"max_context {self.max_context} leaves no room beside {self.mtp_heads} prediction heads")

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "GqaMtpConfig":
        K = cls.KEYS
        n_heads = _take(raw, K["n_heads"], int)
        if any(k in raw for k in K["group_size"]):
            group = _take(raw, K["group_size"], int)
        elif "n_kv_heads" in raw:
            kv = _take(raw, ("n_kv_heads",), int)
            if kv < 1 or n_heads % kv:
                raise ConfigError(f"n_heads {n_heads} is not a multiple of n_kv_heads {kv}")
            group = n_heads // kv
        else:
            raise ConfigError("config.json lacks 'NUM_GROUPS' (query heads per key/value head; also read as "
                              "'group_size' or, as a head count, 'n_kv_heads')")
        used = {n for names in K.values() for n in names} | {"architecture", "n_kv_heads"}
        return cls(
            d_model=_take(raw, K["d_model"], int),
            vocab_size=_take(raw, K["vocab_size"], int),
            max_context=_take(raw, K["max_context"], int),
            rope_base=_take(raw, K["rope_base"], float),
            n_heads=n_heads,
            n_layers=_take(raw, K["n_layers"], int),
            ffn_hidden=_take(raw, K["ffn_hidden"], int),
            group_size=group,
            mtp_heads=_take(raw, K["mtp_heads"], int, 0, required=False),
            rms_eps=_take(raw, K["rms_eps"], float, 2e-8, required=False),
            tie_embeddings=_take(raw, K["tie_embeddings"], bool, True, required=False),
            eos_token_id=_take(raw, K["eos_token_id"], int, -1, required=False),
            architecture=str(raw.get("architecture", "GqaMtpTransformer")),
            extra={k: v for k, v in raw.items() if k not in used},
        )

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"architecture": self.architecture}
        for f in fields(self):
            if f.name in self.KEYS:
                out[self.KEYS[f.name][0]] = getattr(self, f.name)
        return out


def config_from_dict(raw: Mapping[str, Any]):
    if "architecture" not in raw:
        raise ConfigError("config.json lacks 'architecture'; known: " + ", ".join(ARCHITECTURES))
    try:
        arch = ARCHITECTURES.get(str(raw["architecture"]))
    except KeyError as e:
        raise ConfigError(str(e.args[0])) from None
    return arch.config_class.from_dict(raw)


def load_config(model_dir: str):
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"no config.json in {model_dir!r}")
    with open(path) as f:
        try:
            raw = json.load(f)
        except json.JSONDecodeError as e:
            raise ConfigError(f"{path}: not valid JSON ({e})") from None
    if not isinstance(raw, dict):
        raise ConfigError(f"{path}: expected a JSON object")
    return config_from_dict(raw)


def save_config(config, model_dir: str) -> None:
    os.makedirs(model_dir, exist_ok=True)
    with open(os.path.join(model_dir, "config.json"), "w") as f:
        json.dump(config.to_dict(), f, indent=1)
        f.write("\n")

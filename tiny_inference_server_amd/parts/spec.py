"""Plain data that describes a model as an arrangement of parts.

An architecture turns its configuration into a `ModelSpec`; the engine builds
and runs the spec and never asks which architecture it came from.

* `PartSpec`      one part: its role and kind (a registry and a name in it), its sizes and
                  constants, and the full names of the tensors it owns.
* `LayerSpec`     one block: an arrangement kind and the parts it arranges, by the names the arrangement gives them.
* `LayerCall`     one entry of the run order: which layer runs and whose cache it uses.
* `StageSpec`     one pass over the rows of a step: where its input comes from,
                  the ordered calls, the closing norm.  A stage with `lag` j runs
                  at positions j behind the tokens that the step brings.
* `ModelSpec`     the layers, the stages and the shared tables.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Mapping, Optional, Tuple


@dataclass(frozen=True)
class PartSpec:
    role: str                     # which registry `kind` is looked up in: "norm", "position", "mixer",
                                  # "feed_forward" or "stage_input"
    kind: str
    params: Mapping[str, Any] = field(default_factory=dict)    # sizes, constants, nested PartSpecs
    tensors: Mapping[str, str] = field(default_factory=dict)   # local key -> tensor name in the file


@dataclass(frozen=True)
class LayerSpec:
    """One block. Which parts a block has is the arrangement's business: it declares their names, and the loader,
    the cache manager and the graph check walk whatever is there. A block may have no feed-forward, two mixers,
    norms in other places; every part whose role is "mixer" gets a cache of its own if its kind asks for one."""
    arrangement: str                      # block arrangement kind, e.g. "prenorm_residual"
    parts: Mapping[str, PartSpec]         # the arrangement's name for the part -> the part

    def part(self, name: str) -> PartSpec:
        try:
            return self.parts[name]
        except KeyError:
            raise KeyError(f"a {self.arrangement!r} block has no part {name!r}; it has {sorted(self.parts)}") from None

    def with_part(self, name: str, spec: PartSpec) -> "LayerSpec":
        return LayerSpec(self.arrangement, {**self.parts, name: spec})

    def mixers(self) -> Tuple[Tuple[str, PartSpec], ...]:
        return tuple((n, p) for n, p in self.parts.items() if p.role == "mixer")


@dataclass(frozen=True)
class LayerCall:
    layer: int                        # index into ModelSpec.layers
    cache: Optional[str] = None       # cache key; None: a key of this call's own
    writes_cache: bool = True         # False: only reads what the owner of `cache` wrote


@dataclass(frozen=True)
class StageSpec:
    name: str
    lag: int                          # rows of this stage sit `lag` positions behind the step's tokens
    input: PartSpec                   # "token_embedding" or "fuse_previous_stage"
    calls: Tuple[LayerCall, ...]
    out_norm: PartSpec
    state_key: Optional[str] = None   # cache key of the input part's per-request state, if it has one


@dataclass(frozen=True)
class ModelSpec:
    d_model: int
    vocab_size: int
    max_context: int
    layers: Tuple[LayerSpec, ...]
    stages: Tuple[StageSpec, ...]
    embedding: str                    # tensor name of the token table (vocab, d_model)
    lm_head: str                      # tensor name of the output table (vocab, d_model); the same name when tied
    eos_token_id: int = -1
    ignorable: Tuple[str, ...] = ()   # glob patterns of derived buffers a file may also hold


# What a part needs from the cache manager --------------------------------------------------

@dataclass(frozen=True)
class PagedKvNeed:
    """Keys and values of every position (window 0) or of the last `window` positions."""
    n_kv_heads: int
    head_dim: int
    window: int = 0


@dataclass(frozen=True)
class StateNeed:
    """A block of fixed size for each live request."""
    shape: Tuple[int, ...]
    dtype: str = "compute"            # "compute": the engine's dtype; or "float32" / "int32"

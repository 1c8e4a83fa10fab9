"""Registries of part kinds and the interfaces the engine expects of them.

A part is built from a `PartSpec` (its sizes and constants), the tensors it named, and an `ops` object
that carries the kernels, the device and the compute dtype. No part is told which model it belongs to.

Interfaces
----------
every part class
    tensor_shapes(params) -> {local key: shape}        classmethod; what it wants from the weight file
    __init__(spec, tensors, ops)                       tensors.of(spec, key) -> the CPU tensor as stored;
                                                       nested parts are built with build_part(sub_spec, tensors, ops)

norm            __call__(x) -> y                       rows in, rows out
position        rotary() -> (table | None, interleaved)   a table of (cos, sin) per position and pair for
                                                       mixers that rotate queries and keys
                score_slopes(n_heads) -> [n_heads] | None   optional: a bias slope[h] * (key position - row position)
                                                       on the attention scores, for encodings that work there
every part      graph_safe = True                      class attribute, only if what the part launches depends on the
                                                       step's device arrays alone (then decode steps may be captured
                                                       as graphs); absent or False keeps the model on plain launches;
                                                       "single_rows": the promise holds for steps in which every
                                                       request brings one token (those are still captured)
mixer           cache_need(params) -> PagedKvNeed | StateNeed | None      classmethod
                forward(x, ctx, residual=None) -> y    x: normed rows; ctx: CallContext; adds `residual` if given
feed-forward    forward(x, residual=None) -> y
                a mixer or feed-forward with the class attribute fuses_norm = True takes forward(..., norm=part)
                instead: x arrives un-normed and the part applies `norm` itself, fused into its first product
                where it can
arrangement     part_names (the names of the parts it wires), __init__(layer_spec, tensors, ops) (the base class
                builds self.parts), forward(x, ctx) -> x; a mixer part gets ctx.of(its name)
planning        a part may offer plan_key() -> hashable | None and plan_rows(seq_rows, add) -> {name: (array id,
                host values...)}: host-side work lists for its kernels, made once per step and distinct key while the
                step's arrays are packed, found again in batch.extras[name]
stage input     state_need(params) -> StateNeed | None classmethod
                forward(batch, previous_output, previous_batch, shared, state) -> rows
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from ..config.registry import Registry

MIXERS: Registry = Registry("mixer")
FEED_FORWARDS: Registry = Registry("feed-forward")
NORMS: Registry = Registry("norm")
POSITION_ENCODINGS: Registry = Registry("position encoding")
ARRANGEMENTS: Registry = Registry("block arrangement")
STAGE_INPUTS: Registry = Registry("stage input")


@dataclass
class CallContext:
    """What one layer call sees of the step: the rows' metadata and the cache that belongs to the call.

    A block with one mixer finds that mixer's cache right here. A block with several asks `ctx.of(part name)` for
    each mixer's own context (same batch, that part's cache)."""
    batch: Any                       # engine.batch.StageBatch
    group: Optional[str] = None      # page group of the call's cache, for paged needs
    plane: Any = None                # [pages, 2, kv heads, page size, head size] for paged needs
    state: Any = None                # [max requests, *shape] for state needs
    writes_cache: bool = True
    residual_is_spent: bool = False  # the caller will not read the residual it passes again: it may be overwritten
    bindings: Optional[Dict[str, "CallContext"]] = None     # per mixer part of the block

    def of(self, part_name: str) -> "CallContext":
        if self.bindings and part_name in self.bindings:
            return self.bindings[part_name]
        return self


class Arrangement:
    """Base of block arrangements: builds the parts the spec names and checks them against what the class declares.

    part_names: the names this arrangement wires together (None: whatever the spec brings). After construction
    `self.parts[name]` is the built part."""
    part_names: Optional[Tuple[str, ...]] = None

    def __init__(self, layer_spec, tensors, ops):
        if self.part_names is not None and set(layer_spec.parts) != set(self.part_names):
            raise ValueError(f"a {layer_spec.arrangement!r} block is made of {sorted(self.part_names)}, "
                             f"its spec brings {sorted(layer_spec.parts)}")
        self.ops = ops
        self.parts = {name: build_part(spec, tensors, ops) for name, spec in layer_spec.parts.items()}


class Tensors:
    """The loaded tensors by their names in the file; a part asks for its own by local key."""

    def __init__(self, by_name):
        self.by_name = by_name

    def of(self, spec, key):
        try:
            return self.by_name[spec.tensors[key]]
        except KeyError:
            raise KeyError(f"part {spec.kind!r} asks for tensor {key!r} -> {spec.tensors.get(key)!r}, "
                           f"which was not loaded") from None


REGISTRIES = {"mixer": MIXERS, "feed_forward": FEED_FORWARDS, "norm": NORMS, "position": POSITION_ENCODINGS,
              "stage_input": STAGE_INPUTS}


def part_class(spec):
    try:
        registry = REGISTRIES[spec.role]
    except KeyError:
        raise KeyError(f"unknown part role {spec.role!r}; known: {', '.join(sorted(REGISTRIES))}") from None
    return registry.get(spec.kind)


def build_part(spec, tensors, ops):
    return part_class(spec)(spec, tensors, ops)


def expected_tensors(spec):
    """{tensor name in the file: shape} of a part and of the parts nested in its params."""
    out = {}
    shapes = part_class(spec).tensor_shapes(spec.params)
    for key, shape in shapes.items():
        if key not in spec.tensors:
            raise KeyError(f"part {spec.kind!r} needs a tensor name for {key!r}")
        out[spec.tensors[key]] = tuple(int(s) for s in shape)
    for v in spec.params.values():
        if hasattr(v, "role") and hasattr(v, "kind"):
            out.update(expected_tensors(v))
    return out


def normed_linear(ops, x, w, norm, **kw):
    """norm(x) . w^T: through the fused kernel if the norm offers its (gain, eps), else in two steps."""
    if norm is None:
        return ops.linear(x, w, **kw)
    if hasattr(norm, "as_rms"):
        return ops.linear(x, w, rms=norm.as_rms(), **kw)
    return ops.linear(norm(x), w, **kw)


def to_compute(ops, t):
    """A stored matrix as the kernels take it: on the device, in the compute dtype."""
    return t.to(device=ops.device, dtype=ops.dtype).contiguous()


def to_gain(ops, t):
    """A stored 1-d gain on the device in 32-bit (widening bfloat16 is exact)."""
    return t.to(device=ops.device, dtype=__import__("torch").float32).contiguous()

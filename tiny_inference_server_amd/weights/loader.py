"""Weights from a model folder's model.safetensors, by tensor name.

What the model's spec expects is compared with what the file holds before anything is read; every
missing tensor, unexpected tensor and wrong shape is reported in one error. Floating tensors stored in 16
bits are kept as bfloat16, tensors stored in 32 bits stay 32-bit, integer tables become int32. Parts
convert what they feed to the matrix kernels to the compute dtype when they are built.

(The reference loads a training checkpoint positionally, main_models_new.py:234-249; names replace that.)
"""
from __future__ import annotations

import fnmatch
import os
from typing import Dict, Iterable, Mapping, Tuple

import torch

from ..parts.base import expected_tensors as part_tensors


class WeightError(ValueError):
    pass


def spec_tensors(spec) -> Dict[str, Tuple[int, ...]]:
    """{tensor name: shape} of everything a ModelSpec reads from the file."""
    want: Dict[str, Tuple[int, ...]] = {}

    def add(name, shape):
        shape = tuple(int(s) for s in shape)
        if name in want and want[name] != shape:
            raise WeightError(f"the spec asks for tensor {name!r} with two shapes: {want[name]} and {shape}")
        want[name] = shape

    add(spec.embedding, (spec.vocab_size, spec.d_model))
    add(spec.lm_head, (spec.vocab_size, spec.d_model))
    for layer in spec.layers:
        for part in layer.parts.values():
            for n, s in part_tensors(part).items():
                add(n, s)
    for stage in spec.stages:
        for part in (stage.input, stage.out_norm):
            for n, s in part_tensors(part).items():
                add(n, s)
    return want


def _keep_dtype(t: torch.Tensor, name: str) -> torch.Tensor:
    if t.dtype in (torch.bfloat16, torch.float32, torch.int32):
        return t
    if t.dtype == torch.float16:
        return t.to(torch.bfloat16)
    if t.dtype == torch.float64:
        return t.to(torch.float32)
    if t.dtype in (torch.int64, torch.int16, torch.int8, torch.uint8):
        return t.to(torch.int32)
    raise WeightError(f"tensor {name!r} has dtype {t.dtype}, which this engine does not read")


def check_names_and_shapes(want: Mapping[str, Tuple[int, ...]], have: Mapping[str, Tuple[int, ...]],
                           ignorable: Iterable[str], where: str) -> None:
    ignorable = tuple(ignorable)
    missing = sorted(n for n in want if n not in have)
    unexpected = sorted(n for n in have if n not in want and not any(fnmatch.fnmatchcase(n, p) for p in ignorable))
    wrong = sorted((n, have[n], want[n]) for n in want if n in have and tuple(have[n]) != tuple(want[n]))
    if not (missing or unexpected or wrong):
        return
    lines = [f"{where} does not fit the model that its config.json describes:"]
    if missing:
        lines.append(f"  missing tensors ({len(missing)}): " + ", ".join(missing))
    if unexpected:
        lines.append(f"  unexpected tensors ({len(unexpected)}): " + ", ".join(unexpected))
    if wrong:
        lines.append(f"  wrong shapes ({len(wrong)}): " +
                     ", ".join(f"{n} is {list(h)}, expected {list(w)}" for n, h, w in wrong))
    raise WeightError("\n".join(lines))


def load_tensors(model_dir: str, spec) -> Dict[str, torch.Tensor]:
    """All tensors the spec names, on the CPU, checked against the spec first."""
    from safetensors import safe_open

    path = os.path.join(model_dir, "model.safetensors")
    if not os.path.isfile(path):
        raise WeightError(f"no model.safetensors in {model_dir!r}")
    want = spec_tensors(spec)
    with safe_open(path, framework="pt", device="cpu") as f:
        have = {n: tuple(f.get_slice(n).get_shape()) for n in f.keys()}
        check_names_and_shapes(want, have, spec.ignorable, path)
        return {n: _keep_dtype(f.get_tensor(n), n) for n in want}
